// C-ABI entry points of the HIP side (include/pf_moe_hip.h).
#include "pf_moe_internal.h"
#include "pf_moe_debug.h"
#include "../../include/pf_iq2_codes.h"
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <mutex>

static thread_local char g_error[256] = "";

void pf_set_error(const char *what, hipError_t code) {
    snprintf(g_error, sizeof g_error, "%s: %s", what, hipGetErrorString(code));
}
#define HIP_TRY(call)                                                                                   \
    do {                                                                                                \
        hipError_t e_ = (call);                                                                         \
        if (e_ != hipSuccess) { pf_set_error(#call, e_); return PF_HIP_E_RUNTIME; }                     \
    } while (0)

extern "C" const char *pf_hip_last_error(void) { return g_error; }

extern "C" int pf_hip_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

// Scratch of the entry point that allocates nothing (pf_hip_moe_forward_static): one array per GPU,
// held from the library's load until the process ends.  In host code the array's name is only a
// handle for hipGetSymbolAddress; kernels and copies use the address that call returns.
#define PF_STATIC_SCRATCH_BYTES ((size_t)1 << 20)
#define PF_MAX_DEVICES 16
static __device__ __align__(256) unsigned char scratch[PF_STATIC_SCRATCH_BYTES];
static uint8_t *g_scratch_ptr[PF_MAX_DEVICES];

// The current device's copy of the array; looked up once per device, with that device current.
static int static_scratch(uint8_t **out) {
    int dev = -1;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= PF_MAX_DEVICES) {
        snprintf(g_error, sizeof g_error, "device %d is beyond the %d devices the static scratch serves", dev, PF_MAX_DEVICES);
        return PF_HIP_E_UNSUPPORTED;
    }
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        g_scratch_ptr[dev] = static_cast<uint8_t *>(p);
    }
    *out = g_scratch_ptr[dev];
    return PF_HIP_OK;
}

static int need_device(void) {
    if (pf_hip_device_count() >= 1) return PF_HIP_OK;
    snprintf(g_error, sizeof g_error, "no HIP device");
    return PF_HIP_E_NO_DEVICE;
}

// IQ2_XXS constants, one copy per process (one device per process): the 256 x 8
// magnitudes, and for the integer dot products four signed magnitudes per (grid entry,
// sign nibble): words [0, 4096) positions 0..3, words [4096, 8192) positions 4..7.
static uint64_t *g_grid = nullptr;
static uint32_t *g_signed = nullptr;

static bool upload_constants(void) {
    if (g_grid && g_signed) return true;
    uint64_t grid[256];
    uint32_t *tables = (uint32_t *)malloc(8192 * sizeof(uint32_t));
    if (!tables) return false;
    for (unsigned g = 0; g < 256; g++) {
        uint64_t v = 0;
        for (unsigned j = 0; j < 8; j++) v |= (uint64_t)pf_iq2_grid_byte(g, j) << (8 * j);
        grid[g] = v;
        for (unsigned s = 0; s < 16; s++)
            for (unsigned half = 0; half < 2; half++) {
                uint32_t word = 0;
                for (unsigned j = 0; j < 4; j++) {
                    int m = (int)pf_iq2_grid_byte(g, 4 * half + j);
                    if ((s >> j) & 1u) m = -m;
                    word |= ((uint32_t)m & 255u) << (8 * j);
                }
                tables[4096 * half + ((g << 4) | s)] = word;
            }
    }
    uint64_t *dg = nullptr;
    uint32_t *dt = nullptr;
    bool ok = hipMalloc(&dg, sizeof grid) == hipSuccess && hipMalloc(&dt, 8192 * 4) == hipSuccess &&
              hipMemcpy(dg, grid, sizeof grid, hipMemcpyHostToDevice) == hipSuccess &&
              hipMemcpy(dt, tables, 8192 * 4, hipMemcpyHostToDevice) == hipSuccess;
    free(tables);
    if (!ok) {
        if (dg) (void)hipFree(dg);
        if (dt) (void)hipFree(dt);
        return false;
    }
    g_grid = dg;
    g_signed = dt;
    return true;
}
const uint64_t *pf_device_iq2_grid(void) { return upload_constants() ? g_grid : nullptr; }
const uint32_t *pf_device_iq2_signed(void) { return upload_constants() ? g_signed : nullptr; }

static bool block_geometry(uint32_t type, size_t *block, size_t *bytes) { return pf_block_geometry(type, block, bytes); }
static size_t split_header_bytes(uint32_t type) { return pf_split_header_bytes(type); }

// Host bytes into device memory through a page-locked buffer of the library's own (32 MB, allocated
// at the first upload and kept until the process ends), two halves in turn so that the CPU fills
// one while the other is on its way.  The caller's memory (for a checkpoint: a read-only mapping of
// the file) is read by the CPU only and never handed to the runtime, which would otherwise
// page-lock it for the transfer.  Uploads of one process take turns.
struct Bounce {
    static constexpr size_t HALF = (size_t)16 << 20;
    uint8_t *base = nullptr;
    hipEvent_t sent[2] = {nullptr, nullptr};
    bool open() {
        if (base) return true;
        const bool ok = hipHostMalloc((void **)&base, 2 * HALF, hipHostMallocDefault) == hipSuccess &&
                        hipEventCreate(&sent[0]) == hipSuccess && hipEventCreate(&sent[1]) == hipSuccess;
        if (!ok) base = nullptr;
        return ok;
    }
    hipError_t upload(void *d_dst, const void *src, size_t bytes) {
        hipError_t e = hipSuccess;
        bool busy[2] = {false, false};
        int k = 0;
        for (size_t at = 0; at < bytes && e == hipSuccess; k ^= 1) {
            const size_t n = bytes - at < HALF ? bytes - at : HALF;
            if (busy[k]) e = hipEventSynchronize(sent[k]);
            if (e != hipSuccess) break;
            memcpy(base + k * HALF, static_cast<const uint8_t *>(src) + at, n);
            e = hipMemcpyAsync(static_cast<uint8_t *>(d_dst) + at, base + k * HALF, n, hipMemcpyHostToDevice, nullptr);
            if (e == hipSuccess) e = hipEventRecord(sent[k], nullptr);
            busy[k] = true;
            at += n;
        }
        const hipError_t done = hipStreamSynchronize(nullptr);   // the buffer is free again when this returns
        return e != hipSuccess ? e : done;
    }
};

static hipError_t upload_from_host(void *d_dst, const void *src, size_t bytes) {
    static std::mutex turn;
    static Bounce *bounce = new Bounce();   // never freed: the runtime may be gone when statics are destroyed
    std::lock_guard<std::mutex> hold(turn);
    if (!bounce->open()) return hipErrorOutOfMemory;
    return bounce->upload(d_dst, src, bytes);
}

extern "C" int pf_hip_moe_create(const PfHipMoeDesc *desc, const void *const host_weights[8], const size_t bytes[8],
                                 PfHipMoe **out) {
    if (out) *out = nullptr;
    if (!desc || !host_weights || !bytes || !out) return PF_HIP_E_ARGUMENT;
    if (need_device()) return PF_HIP_E_NO_DEVICE;
    const size_t h = desc->hidden, i = desc->inter, s = desc->shared_inter, E = desc->experts;
    const size_t k_storage[8] = {h, h, h, desc->down_physical, h, h, s, h};
    const size_t k_logical[8] = {h, h, h, i, h, h, s, h};
    const size_t n_out[8] = {E, i, i, h, s, s, h, 1};
    const size_t experts[8] = {1, E, E, E, 1, 1, 1, 1};
    if (!h || !i || !s || !E || !desc->top_k || desc->top_k > E || desc->down_physical < i) return PF_HIP_E_ARGUMENT;
    if (desc->type[0] != PF_F32 || desc->type[7] != PF_F32) return PF_HIP_E_UNSUPPORTED;
    PfHipMoe *m = (PfHipMoe *)calloc(1, sizeof *m);
    if (!m) return PF_HIP_E_MEMORY;
    m->desc = *desc;
    size_t gguf_bytes[8];
    for (int a = 0; a < 8; a++) {
        PfTensorPlace place;
        if (k_storage[a] > 0x7fffffffu || n_out[a] > 0x7fffffffu ||
            !pf_tensor_place(desc->type[a], k_storage[a], n_out[a], experts[a], &place)) {
            pf_hip_moe_destroy(m);
            return PF_HIP_E_UNSUPPORTED;
        }
        gguf_bytes[a] = place.gguf_bytes;
        // a layer whose routed tensors stay on disk (forwards then read them from an expert pool): all three absent
        const bool routed = a >= 1 && a <= 3;
        if (routed && !host_weights[1] && !host_weights[2] && !host_weights[3]) m->streamed = true;
        else if (bytes[a] < gguf_bytes[a] || !host_weights[a]) { pf_hip_moe_destroy(m); return PF_HIP_E_ARGUMENT; }
        m->k_logical[a] = (int)k_logical[a];
        m->n_out[a] = place.n_out;
        m->blocks_per_row[a] = place.blocks_per_row;
        m->row_bytes[a] = place.row_bytes;
        m->scale_offset[a] = place.scale_offset;
        m->bytes[a] = place.bytes;
        m->expert_bytes[a] = place.expert_bytes;
    }
    if (!upload_constants()) { pf_hip_moe_destroy(m); return PF_HIP_E_MEMORY; }
    {   // set-up: this device's address of the static scratch, so that the entry point that uses it calls nothing but launches
        uint8_t *unused = nullptr;
        const int rc = static_scratch(&unused);
        if (rc != PF_HIP_OK) { pf_hip_moe_destroy(m); return rc; }
    }
    m->iq2_grid = g_grid;
    m->iq2_signed = g_signed;
    for (int a = 0; a < 8; a++) {
        if (m->streamed && a >= 1 && a <= 3) continue;
        hipError_t e = hipMalloc((void **)&m->w[a], m->bytes[a]);
        const size_t head = split_header_bytes(desc->type[a]);
        if (e == hipSuccess && head) {
            uint8_t *staging = nullptr;
            size_t block, size;
            block_geometry(desc->type[a], &block, &size);
            e = hipMalloc((void **)&staging, gguf_bytes[a]);
            if (e == hipSuccess) e = upload_from_host(staging, host_weights[a], gguf_bytes[a]);
            if (e == hipSuccess) {
                if (desc->type[a] == PF_IQ2_XXS)
                    pf_launch_iq2_split(staging, m->w[a], reinterpret_cast<uint16_t *>(m->w[a] + m->scale_offset[a]),
                                        gguf_bytes[a] / 66, nullptr);
                else
                    pf_launch_block_split(staging, m->w[a], m->w[a] + m->scale_offset[a], gguf_bytes[a] / size,
                                          (int)size, (int)head, nullptr);
                e = hipDeviceSynchronize();
            }
            if (staging) (void)hipFree(staging);
        } else if (e == hipSuccess) {
            e = upload_from_host(m->w[a], host_weights[a], m->bytes[a]);
        }
        if (e != hipSuccess) {
            pf_set_error("weight upload", e);
            pf_hip_moe_destroy(m);
            return e == hipErrorOutOfMemory ? PF_HIP_E_MEMORY : PF_HIP_E_RUNTIME;
        }
        m->total_bytes += m->bytes[a];
    }
    if (pf_route_needs_slabs((int)E, (int)desc->top_k)) {   // router copy in 64-expert slabs: only where every token is routed in serial order
        const size_t slab_floats = pf_router_slab_floats((int)E, (int)h);
        hipError_t e = hipMalloc((void **)&m->router_t, slab_floats * sizeof(float));
        if (e == hipSuccess) {
            pf_launch_router_slabs(reinterpret_cast<const float *>(m->w[0]), (int)E, (int)h, m->router_t, nullptr);
            e = hipDeviceSynchronize();
        }
        if (e != hipSuccess) {
            pf_set_error("router copy", e);
            pf_hip_moe_destroy(m);
            return e == hipErrorOutOfMemory ? PF_HIP_E_MEMORY : PF_HIP_E_RUNTIME;
        }
        m->total_bytes += slab_floats * sizeof(float);
    }
    m->decode_ready = !m->streamed && pf_decode_supported(*desc);
    // prefill path: squared norms of the router rows (the routing tolerance's bound)
    m->prefill_ready = !m->streamed && pf_prefill_supported(*desc);
    if (m->prefill_ready) {
        hipError_t e = hipMalloc((void **)&m->w_norm2, E * sizeof(float));
        if (e == hipSuccess) {
            pf_launch_row_norm2(reinterpret_cast<const float *>(m->w[0]), (int)E, (int)h, m->w_norm2, nullptr);
            e = hipDeviceSynchronize();
        }
        if (e != hipSuccess) {
            pf_set_error("prefill constants", e);
            pf_hip_moe_destroy(m);
            return e == hipErrorOutOfMemory ? PF_HIP_E_MEMORY : PF_HIP_E_RUNTIME;
        }
        // Second, tile-ordered copy of the expert tensors: the grouped product then reads whole cache
        // lines once instead of 32-byte pieces of lines it meets again a stage later.  It doubles the
        // expert bytes; PF_MOE_PREFILL_COPY=0 does without it (the same kernels read the row order).
        const char *copy = getenv("PF_MOE_PREFILL_COPY");
        if (!copy || strcmp(copy, "0") != 0) {
            for (int a = 1; a <= 6 && e == hipSuccess; a++) {
                if (desc->type[a] != PF_Q4_K) continue;
                e = hipMalloc((void **)&m->w_tiled[a], m->bytes[a]);
                if (e == hipSuccess) {
                    pf_launch_q4k_tile(m->w[a], m->w_tiled[a], (size_t)n_out[a] * experts[a], m->blocks_per_row[a], nullptr);
                    m->total_bytes += m->bytes[a];
                }
            }
            if (e == hipSuccess) e = hipDeviceSynchronize();
            if (e != hipSuccess) {
                pf_set_error("tile-ordered weights", e);
                pf_hip_moe_destroy(m);
                return e == hipErrorOutOfMemory ? PF_HIP_E_MEMORY : PF_HIP_E_RUNTIME;
            }
        }
    }
    {   // Tile-ordered second copies for the decode kernels whose lanes are weight rows: the IQ2_XXS expert tensors (all
        // six of a layer that is IQ2_XXS throughout; the routed gate and up of the q2 checkpoint profile) and the Q8_0
        // shared gate and up of both profiles.  PF_MOE_PREFILL_COPY=0 does without them, as for Q4_K.
        const char *copy = getenv("PF_MOE_PREFILL_COPY");
        bool all_iq2 = true;
        for (int a = 1; a <= 6; a++) all_iq2 &= desc->type[a] == PF_IQ2_XXS;
        hipError_t e = hipSuccess;
        if (m->decode_ready && (!copy || strcmp(copy, "0") != 0)) {
            for (int a = 1; a <= 6 && e == hipSuccess; a++) {
                const bool gate_or_up = a == 1 || a == 2 || a == 4 || a == 5;
                if (n_out[a] % 32) continue;
                if (desc->type[a] == PF_IQ2_XXS && (all_iq2 || a == 1 || a == 2)) {
                    const size_t bytes = pf_i2t_expert_bytes((int)n_out[a], m->blocks_per_row[a]) * experts[a];
                    e = hipMalloc((void **)&m->w_itile[a], bytes);
                    if (e == hipSuccess) {
                        pf_launch_iq2_tile(m->w[a], reinterpret_cast<const uint16_t *>(m->w[a] + m->scale_offset[a]), m->w_itile[a],
                                           (size_t)n_out[a] * experts[a], m->blocks_per_row[a], nullptr);
                        m->total_bytes += bytes;
                    }
                } else if (desc->type[a] == PF_Q8_0 && gate_or_up && experts[a] == 1 && k_storage[a] % 64 == 0) {
                    const size_t bytes = pf_q8t_expert_bytes((int)n_out[a], (int)(k_storage[a] / 64));
                    e = hipMalloc((void **)&m->w_qtile[a], bytes);
                    if (e == hipSuccess) {
                        pf_launch_q8_tile(m->w[a], reinterpret_cast<const uint16_t *>(m->w[a] + m->scale_offset[a]), m->w_qtile[a],
                                          n_out[a], m->blocks_per_row[a], nullptr);
                        m->total_bytes += bytes;
                    }
                }
            }
            if (e == hipSuccess) e = hipDeviceSynchronize();
            if (e != hipSuccess) {
                pf_set_error("tile-ordered weights", e);
                pf_hip_moe_destroy(m);
                return e == hipErrorOutOfMemory ? PF_HIP_E_MEMORY : PF_HIP_E_RUNTIME;
            }
        }
    }
    // A streamed layer that is Q4_K throughout, or in the q4 checkpoint profile (Q4_K gate and up, MXFP4 down, Q8_0 shared
    // expert): tile-ordered copies of its shared expert's tensors as the resident layer keeps them, so that short batches
    // run the tile decode kernels on pool slots (Q4_K slots in tile order; the routed tensors are not here to be copied).
    if (m->streamed) {
        bool all_q4k = true, all_iq2 = true;
        bool q4_profile = desc->type[1] == PF_Q4_K && desc->type[2] == PF_Q4_K && desc->type[3] == PF_MXFP4;
        bool q2_profile = desc->type[1] == PF_IQ2_XXS && desc->type[2] == PF_IQ2_XXS && desc->type[3] == PF_Q2_K;
        for (int a = 1; a <= 6; a++) { all_q4k &= desc->type[a] == PF_Q4_K; all_iq2 &= desc->type[a] == PF_IQ2_XXS; }
        for (int a = 4; a <= 6; a++) { q4_profile &= desc->type[a] == PF_Q8_0; q2_profile &= desc->type[a] == PF_Q8_0; }
        const int combination = all_q4k ? 1 : all_iq2 ? 2 : q2_profile ? 3 : q4_profile ? 4 : 0;
        const char *copy = getenv("PF_MOE_PREFILL_COPY");
        if (combination && pf_decode_supported(*desc) && (!copy || strcmp(copy, "0") != 0)) {
            hipError_t e = hipSuccess;
            for (int a = 4; a <= 6 && e == hipSuccess && combination == 1; a++) {
                if (n_out[a] % 32) { e = hipErrorInvalidValue; break; }
                e = hipMalloc((void **)&m->w_tiled[a], m->bytes[a]);
                if (e == hipSuccess) {
                    pf_launch_q4k_tile(m->w[a], m->w_tiled[a], (size_t)n_out[a], m->blocks_per_row[a], nullptr);
                    m->total_bytes += m->bytes[a];
                }
            }
            for (int a = 4; a <= 6 && e == hipSuccess && combination == 2; a++) {
                if (n_out[a] % 32) { e = hipErrorInvalidValue; break; }
                const size_t bytes = pf_i2t_expert_bytes((int)n_out[a], m->blocks_per_row[a]);
                e = hipMalloc((void **)&m->w_itile[a], bytes);
                if (e == hipSuccess) {
                    pf_launch_iq2_tile(m->w[a], reinterpret_cast<const uint16_t *>(m->w[a] + m->scale_offset[a]), m->w_itile[a],
                                       (size_t)n_out[a], m->blocks_per_row[a], nullptr);
                    m->total_bytes += bytes;
                }
            }
            for (int a = 4; a <= 5 && e == hipSuccess && (combination == 4 || combination == 3); a++) {
                if (n_out[a] % 32 || k_storage[a] % 64) { e = hipErrorInvalidValue; break; }
                const size_t bytes = pf_q8t_expert_bytes((int)n_out[a], (int)(k_storage[a] / 64));
                e = hipMalloc((void **)&m->w_qtile[a], bytes);
                if (e == hipSuccess) {
                    pf_launch_q8_tile(m->w[a], reinterpret_cast<const uint16_t *>(m->w[a] + m->scale_offset[a]), m->w_qtile[a],
                                      n_out[a], m->blocks_per_row[a], nullptr);
                    m->total_bytes += bytes;
                }
            }
            if (e == hipSuccess) e = hipDeviceSynchronize();
            if (e == hipSuccess) {
                const uint8_t *tiled[8], *itiled[8];   // 1..3: any non-null address stands for the pool's at forward time
                for (int a = 0; a < 8; a++) {
                    const bool routed = a >= 1 && a <= 3;
                    tiled[a] = routed && desc->type[a] == PF_Q4_K ? m->w[0] : m->w_tiled[a];
                    itiled[a] = routed && desc->type[a] == PF_IQ2_XXS ? m->w[0] : m->w_itile[a];
                }
                const bool slots_tile = n_out[1] % 32 == 0 && (combination >= 3 || n_out[3] % 32 == 0);
                if (slots_tile && pf_decode_tile_layer(m->desc, tiled, itiled, m->w_qtile) == combination) m->stream_decode = combination;
            } else {
                (void)hipGetLastError();   // without the copies the general kernels serve every batch
                for (int a = 4; a <= 6; a++) {
                    if (m->w_tiled[a]) { (void)hipFree(m->w_tiled[a]); m->w_tiled[a] = nullptr; }
                    if (m->w_itile[a]) { (void)hipFree(m->w_itile[a]); m->w_itile[a] = nullptr; }
                    if (m->w_qtile[a]) { (void)hipFree(m->w_qtile[a]); m->w_qtile[a] = nullptr; }
                }
            }
        }
    }
    // A Q4_K layer that every kernel family can read through the tile-ordered copy alone (the decode kernels whose lanes
    // are weight rows, the grouped product, the general kernels' tile reader) gives its row-ordered expert tensors
    // back: one copy of the experts in device memory, not two.
    if (pf_decode_tile_layer(m->desc, m->w_tiled, m->w_itile, m->w_qtile) == 1) {
        for (int a = 1; a <= 6; a++) {
            (void)hipFree(m->w[a]);
            m->w[a] = nullptr;
            m->total_bytes -= m->bytes[a];
        }
    }
    *out = m;
    return PF_HIP_OK;
}

extern "C" void pf_hip_moe_destroy(PfHipMoe *m) {
    if (!m) return;
    for (int a = 0; a < 8; a++) if (m->w[a]) (void)hipFree(m->w[a]);
    if (m->w_norm2) (void)hipFree(m->w_norm2);
    if (m->router_t) (void)hipFree(m->router_t);
    for (int a = 0; a < 8; a++) if (m->w_tiled[a]) (void)hipFree(m->w_tiled[a]);
    for (int a = 0; a < 8; a++) if (m->w_itile[a]) (void)hipFree(m->w_itile[a]);
    for (int a = 0; a < 8; a++) if (m->w_qtile[a]) (void)hipFree(m->w_qtile[a]);
    free(m);
}

extern "C" size_t pf_hip_moe_bytes(const PfHipMoe *m) { return m ? m->total_bytes : 0; }

// workspace layout: buffers carved from one allocation, each 256-byte aligned
// (the error word, the ids and the route weights follow each other: a short batch's are fetched by one copy)
enum { W_LOGITS, W_SSQ, W_ERR, W_IDS, W_RW, W_ACT, W_SACT, W_SSCALE, W_X, W_Y, W_SLOTS, W_UNIQ, W_EXACT, W_FLAGS, W_XIMG, W_AIMG,
       W_FLINES, W_FGEN, W_X16, W_ACT16, W_SACT16, W_XSCALE, W_ACTSCALE, W_SACTSCALE, W_XMAX2, W_DOWN, W_COUNTS, W_OFFSETS,
       W_P2R, W_R2P, W_GROUPBAD, W_TILES, W_COUNT };
#define PF_GUARD_BYTES 4096
struct Carve { size_t offset[W_COUNT], size[W_COUNT], total; bool fused; size_t guard; };
// fused: plan the activation lines of the decode path's one-launch expert stage (a workspace of the library's own;
// the static scratch is too small for them and its forwards run the three kernels)
static Carve plan_work(const PfHipMoeDesc *d, size_t cap, bool fused = false, size_t guard = 0) {
    Carve c;
    memset(&c, 0, sizeof c);
    const size_t T = cap ? cap : 1, E = d->experts, K = d->top_k, H = d->hidden, I = d->inter;
    const size_t Td = T < PF_DECODE_MAX_TOKENS ? T : PF_DECODE_MAX_TOKENS;   // tokens per decode launch
    // ... and per launch of the kernels for tile-ordered Q4_K (whether the copies are kept is not known here)
    // (one format throughout, or a checkpoint profile: Q8_0 shared expert)
    bool one_format = (d->type[1] == PF_Q4_K || d->type[1] == PF_IQ2_XXS) && d->type[2] == d->type[1];
    for (int t = 4; t <= 6; t++) one_format &= d->type[t] == d->type[1] || d->type[t] == PF_Q8_0;
    const size_t Tt = !one_format ? Td : T < PF_TILE_DECODE_MAX_TOKENS ? T : PF_TILE_DECODE_MAX_TOKENS;
    size_t want[W_COUNT];
    want[W_LOGITS] = T * E * 4;
    want[W_SSQ] = T * E * 4;
    want[W_RW] = T * K * 4;
    want[W_ACT] = (T * K > Td * K * Td ? T * K : Td * K * Td) * I * 4;
    want[W_SACT] = T * d->shared_inter * 4;
    want[W_SSCALE] = T * 4;
    want[W_X] = T * H * 4;
    want[W_Y] = T * H * 4;
    want[W_IDS] = T * K * 4;
    want[W_SLOTS] = T * K * 4;   // expert streaming: the pairs' pool slots
    want[W_UNIQ] = (1 + 3 * Td * K) * 4;
    want[W_ERR] = 256;
    want[W_EXACT] = 256;
    want[W_FLAGS] = (T + 1) * 4;
    {
        size_t lines = 0;
        if (fused) pf_decode_fused_scratch(*d, &lines);
        want[W_FLINES] = lines;
        want[W_FGEN] = lines ? 256 : 0;
        c.fused = lines != 0;
    }
    {   // digit images of the decode path: the token rows; the activation rows of every (unique expert, token) and the shared expert's
        const size_t widest = I > d->shared_inter ? I : d->shared_inter;
        const size_t rows = Td * K * Td + Td > Tt * (K + 1) ? Td * K * Td + Td : Tt * (K + 1);
        want[W_XIMG] = Tt * pf_image2_words(H) * 4;
        want[W_AIMG] = rows * pf_image2_words(widest) * 4;
    }
    // prefill path: fp16 copies, per-row scales, down products in expert order, grouping tables
    const bool prefill = T > PF_DECODE_MAX_TOKENS && pf_prefill_supported(*d);
    const size_t Tp = prefill ? T : 0, Is = d->shared_inter;
    // one more row each, never written after the workspace's initial memset: the all-zero row
    want[W_X16] = prefill ? (Tp + 1) * pf_prefill_half_row((int)H) * 2 : 0;
    want[W_ACT16] = prefill ? (Tp * K + 1) * pf_prefill_half_row((int)I) * 2 : 0;
    want[W_SACT16] = prefill ? (Tp + 1) * pf_prefill_half_row((int)Is) * 2 : 0;
    want[W_XSCALE] = Tp * 4;
    want[W_ACTSCALE] = Tp * K * 4;
    want[W_SACTSCALE] = Tp * 4;
    want[W_XMAX2] = Tp * 4;
    want[W_DOWN] = (Tp * K + Tp) * H * 4;
    want[W_COUNTS] = prefill ? E * 4 : 0;
    want[W_OFFSETS] = prefill ? (E + 1) * 4 : 0;
    want[W_P2R] = Tp * K * 4;
    want[W_R2P] = Tp * K * 4;
    want[W_GROUPBAD] = prefill ? 4 : 0;
    want[W_TILES] = prefill ? (1 + (size_t)pf_prefill_max_tiles((int)T, (int)E, (int)K)) * 4 : 0;
    c.guard = guard;
    for (int j = 0; j < W_COUNT; j++) {
        c.offset[j] = c.total;
        c.size[j] = (want[j] + 255) & ~(size_t)255;
        c.total += c.size[j] + guard;   // (diagnostics: a guard of a fixed pattern behind every buffer)
    }
    return c;
}

// PF_MOE_DECODE_FUSED=1: one-token forwards of layers the fused launch takes run two launches instead of the three decode
// kernels (measured slower on this GPU: the hand-off through memory inside the launch costs what the kernel boundary does)
static bool fused_wanted() {
    const char *v = getenv("PF_MOE_DECODE_FUSED");
    return v && v[0] == '1';
}

extern "C" size_t pf_hip_work_bytes(const PfHipMoeDesc *desc, size_t token_cap) {
    return desc ? plan_work(desc, token_cap, fused_wanted()).total : 0;
}

static void carve_work(PfHipWork *w, const Carve &c, uint8_t *base);

// The pinned block of a workspace: a head that mirrors the workspace from the error word to the route weights of a short
// batch (one copy brings all three when that span is at most PF_HOST_HEAD_BYTES; ids and weights have places of their
// own for workspaces of more tokens), then input rows, output rows and pool slots of up to PF_HOST_BLOCK_TOKENS
// tokens, each part 256-byte aligned.  The kernels write the output rows straight into the block.
#define PF_HOST_BLOCK_TOKENS PF_TILE_DECODE_MAX_TOKENS
#define PF_HOST_HEAD_BYTES (32 * 1024)
struct HostBlock {
    uint8_t *head;
    uint32_t *ids, *slots;
    float *x, *y, *weights;
    size_t y_offset, bytes;
};
static HostBlock host_block(const PfHipMoeDesc *d, uint8_t *base) {
    const size_t T = PF_HOST_BLOCK_TOKENS, rows = (T * d->hidden * 4 + 255) & ~(size_t)255, pairs = (T * d->top_k * 4 + 255) & ~(size_t)255;
    HostBlock b;
    size_t at = 0;
    b.head = base + at; at += PF_HOST_HEAD_BYTES;
    b.x = (float *)(base + at); at += rows;
    b.y_offset = at;
    b.y = (float *)(base + at); at += rows;
    b.ids = (uint32_t *)(base + at); at += pairs;
    b.weights = (float *)(base + at); at += pairs;
    b.slots = (uint32_t *)(base + at); at += pairs;
    b.bytes = at;
    return b;
}
static size_t host_block_bytes(const PfHipMoeDesc *d) { return host_block(d, nullptr).bytes; }
static bool through_host_block(const PfHipWork *w, size_t tokens) { return w->host && tokens <= PF_HOST_BLOCK_TOKENS; }

// Enqueues the copies that bring a short batch's error word, ids and route weights into the block; after the stream
// has been waited for, host_results hands them out.
struct HostResults { const uint32_t *error_word, *ids; const float *weights; };
static hipError_t fetch_results(const PfHipWork *w, const HostBlock &b, size_t tokens, bool want_ids, bool want_weights,
                                HostResults *r) {
    const size_t pairs = tokens * w->moe->desc.top_k * 4;
    const size_t ids_at = (size_t)((const uint8_t *)w->ids - (const uint8_t *)w->error_word);
    const size_t rw_at = (size_t)((const uint8_t *)w->route_weights - (const uint8_t *)w->error_word);
    r->error_word = (const uint32_t *)b.head;
    if ((const uint8_t *)w->ids > (const uint8_t *)w->error_word && w->route_weights > (const float *)w->ids &&
        rw_at + pairs <= PF_HOST_HEAD_BYTES) {
        const size_t span = want_weights ? rw_at + pairs : want_ids ? ids_at + pairs : 4;
        r->ids = (const uint32_t *)(b.head + ids_at);
        r->weights = (const float *)(b.head + rw_at);
        return hipMemcpyAsync(b.head, w->error_word, span, hipMemcpyDeviceToHost, nullptr);
    }
    r->ids = b.ids;
    r->weights = b.weights;
    hipError_t e = hipMemcpyAsync(b.head, w->error_word, 4, hipMemcpyDeviceToHost, nullptr);
    if (e == hipSuccess && want_ids) e = hipMemcpyAsync(b.ids, w->ids, pairs, hipMemcpyDeviceToHost, nullptr);
    if (e == hipSuccess && want_weights) e = hipMemcpyAsync(b.weights, w->route_weights, pairs, hipMemcpyDeviceToHost, nullptr);
    return e;
}

static void rows_in(void *dst, const void *src, size_t src_pitch, size_t row_bytes, size_t rows) {
    for (size_t r = 0; r < rows; r++) memcpy((uint8_t *)dst + r * row_bytes, (const uint8_t *)src + r * src_pitch, row_bytes);
}
static void rows_out(void *dst, size_t dst_pitch, const void *src, size_t row_bytes, size_t rows) {
    for (size_t r = 0; r < rows; r++) memcpy((uint8_t *)dst + r * dst_pitch, (const uint8_t *)src + r * row_bytes, row_bytes);
}

extern "C" int pf_hip_work_create(const PfHipMoe *moe, size_t token_cap, PfHipWork **out) {
    if (out) *out = nullptr;
    if (!moe || !out) return PF_HIP_E_ARGUMENT;
    PfHipWork *w = (PfHipWork *)calloc(1, sizeof *w);
    if (!w) return PF_HIP_E_MEMORY;
    const char *guard_env = getenv("PF_WORK_GUARD");
    const Carve c = plan_work(&moe->desc, token_cap, fused_wanted(), guard_env && guard_env[0] == '1' ? PF_GUARD_BYTES : 0);
    uint8_t *base = nullptr;
    hipError_t e = hipMalloc((void **)&base, c.total);
    if (e == hipSuccess) e = hipMemset(base, 0, c.total);
    for (int j = 0; j < W_COUNT && c.guard && e == hipSuccess; j++) e = hipMemset(base + c.offset[j] + c.size[j], 0xA5, c.guard);
    if (e != hipSuccess) {
        pf_set_error("workspace allocation", e);
        if (base) (void)hipFree(base);
        free(w);
        return PF_HIP_E_MEMORY;
    }
    w->moe = moe; w->cap = token_cap; w->bytes = c.total;
    carve_work(w, c, base);
    w->guard = c.guard;
    for (int j = 0; j < W_COUNT; j++) w->guard_at[j] = c.offset[j] + c.size[j];
    // short batches through host pointers stage their rows in pinned memory: the copies are then enqueued and the call
    // waits once, for the last of them (without the block the forwards fall back to one blocking copy per buffer)
    if (hipHostMalloc((void **)&w->host, host_block_bytes(&moe->desc), hipHostMallocDefault) != hipSuccess) {
        (void)hipGetLastError();
        w->host = nullptr;
    } else if (hipHostGetDevicePointer((void **)&w->host_device, w->host, 0) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipHostFree(w->host);
        w->host = nullptr;
    }
    *out = w;
    return PF_HIP_OK;
}

static void carve_work(PfHipWork *w, const Carve &c, uint8_t *base) {
    w->logits = (float *)(base + c.offset[W_LOGITS]);
    w->logit_ssq = (float *)(base + c.offset[W_SSQ]);
    w->route_weights = (float *)(base + c.offset[W_RW]);
    w->act = (float *)(base + c.offset[W_ACT]);
    w->shared_act = (float *)(base + c.offset[W_SACT]);
    w->shared_scale = (float *)(base + c.offset[W_SSCALE]);
    w->x = (float *)(base + c.offset[W_X]);
    w->y = (float *)(base + c.offset[W_Y]);
    w->ids = (uint32_t *)(base + c.offset[W_IDS]);
    w->uniq = (uint32_t *)(base + c.offset[W_UNIQ]);
    w->slots = (uint32_t *)(base + c.offset[W_SLOTS]);
    w->error_word = (uint32_t *)(base + c.offset[W_ERR]);
    w->exact_rows = (uint32_t *)(base + c.offset[W_EXACT]);
    w->route_flags = (uint32_t *)(base + c.offset[W_FLAGS]);
    w->ximg = (uint32_t *)(base + c.offset[W_XIMG]);
    w->aimg = (uint32_t *)(base + c.offset[W_AIMG]);
    if (c.fused) {
        w->fuse_lines = (uint32_t *)(base + c.offset[W_FLINES]);
        w->fuse_gen = (uint32_t *)(base + c.offset[W_FGEN]);
    }
    if (c.offset[W_GROUPBAD] != c.offset[W_X16]) {   // the prefill buffers were planned
        w->x16 = (uint16_t *)(base + c.offset[W_X16]);
        w->act16 = (uint16_t *)(base + c.offset[W_ACT16]);
        w->sact16 = (uint16_t *)(base + c.offset[W_SACT16]);
        w->x_scale = (float *)(base + c.offset[W_XSCALE]);
        w->act_scale = (float *)(base + c.offset[W_ACTSCALE]);
        w->sact_scale = (float *)(base + c.offset[W_SACTSCALE]);
        w->x_max2 = (float *)(base + c.offset[W_XMAX2]);
        w->down = (float *)(base + c.offset[W_DOWN]);
        w->counts = (uint32_t *)(base + c.offset[W_COUNTS]);
        w->offsets = (uint32_t *)(base + c.offset[W_OFFSETS]);
        w->pair_to_row = (uint32_t *)(base + c.offset[W_P2R]);
        w->row_to_pair = (uint32_t *)(base + c.offset[W_R2P]);
        w->group_bad = (uint32_t *)(base + c.offset[W_GROUPBAD]);
        w->tiles = (uint32_t *)(base + c.offset[W_TILES]);
    }
}

extern "C" void pf_hip_work_destroy(PfHipWork *w) {
    if (!w) return;
    if (w->logits) (void)hipFree(w->logits);   // base of the single allocation
    if (w->host) (void)hipHostFree(w->host);
    free(w);
}

extern "C" const uint32_t *pf_hip_work_ids(const PfHipWork *w) { return w ? w->ids : nullptr; }
extern "C" const float *pf_hip_work_route_weights(const PfHipWork *w) { return w ? w->route_weights : nullptr; }
extern "C" const float *pf_hip_work_logits(const PfHipWork *w) { return w ? w->logits : nullptr; }
extern "C" const uint32_t *pf_hip_work_error_word(const PfHipWork *w) { return w ? w->error_word : nullptr; }

extern "C" int pf_hip_work_exact_rows(PfHipWork *w, uint32_t *count) {
    if (!w || !count) return PF_HIP_E_ARGUMENT;
    HIP_TRY(hipMemcpy(count, w->exact_rows, 4, hipMemcpyDeviceToHost));
    return PF_HIP_OK;
}

extern "C" int pf_hip_work_full_reroutes(PfHipWork *w, uint32_t *count) {
    if (!w || !count) return PF_HIP_E_ARGUMENT;
    HIP_TRY(hipMemcpy(count, w->exact_rows + 1, 4, hipMemcpyDeviceToHost));
    return PF_HIP_OK;
}

#ifdef PF_TIMING
// instrumented builds only: the router kernel's start and the fused launch's phase stamps (eight per workgroup, 256 workgroups)
extern "C" int pf_debug_stamps(PfHipWork *w, unsigned long long *out) {
    if (!w || !out) return PF_HIP_E_ARGUMENT;
    HIP_TRY(hipMemcpy(out, w->exact_rows + 2, 8, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(out + 1, w->act, 256 * 8 * 8, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemset(w->act, 0, 256 * 8 * 8));
    return PF_HIP_OK;
}
#endif

extern "C" int pf_hip_work_clear_status(PfHipWork *w) {
    if (!w) return PF_HIP_E_ARGUMENT;
    HIP_TRY(hipMemset(w->error_word, 0, 4));
    HIP_TRY(hipMemset(w->exact_rows, 0, 8));
    return PF_HIP_OK;
}

extern "C" int pf_hip_work_check_guards(PfHipWork *w, int *damaged, int *first) {
    if (!w || !damaged || !first) return PF_HIP_E_ARGUMENT;
    *damaged = 0;
    *first = -1;
    if (!w->guard) return PF_HIP_OK;
    HIP_TRY(hipDeviceSynchronize());
    uint8_t *host = (uint8_t *)malloc(w->guard);
    if (!host) return PF_HIP_E_MEMORY;
    const uint8_t *base = (const uint8_t *)w->logits;   // the single allocation starts with its first buffer
    for (int j = 0; j < W_COUNT; j++) {
        if (hipMemcpy(host, base + w->guard_at[j], w->guard, hipMemcpyDeviceToHost) != hipSuccess) { free(host); return PF_HIP_E_RUNTIME; }
        bool intact = true;
        for (size_t b = 0; b < w->guard; b++) intact &= host[b] == 0xA5;
        if (!intact) {
            if (*first < 0) *first = j;
            ++*damaged;
        }
    }
    free(host);
    return PF_HIP_OK;
}

extern "C" void pf_hip_work_force_general(PfHipWork *w, int on) { if (w) w->force_general = on; }
extern "C" void pf_hip_work_limit_kernels(PfHipWork *w, int count) { if (w) w->stage_limit = count > 0 ? count : 0; }

static PfKernelArgs make_args(const PfHipMoe *m, PfHipWork *w, const float *d_x, size_t x_pitch, float *d_y,
                              size_t y_pitch) {
    PfKernelArgs a;
    memset(&a, 0, sizeof a);
    const PfHipMoeDesc *d = &m->desc;
    a.hidden = (int)d->hidden; a.experts = (int)d->experts; a.top_k = (int)d->top_k; a.inter = (int)d->inter;
    a.shared_inter = (int)d->shared_inter; a.down_physical = (int)d->down_physical; a.norm_topk = (int)d->norm_topk;
    for (int j = 0; j < 8; j++) {
        a.type[j] = d->type[j];
        a.w[j] = m->w[j];
        a.row_bytes[j] = m->row_bytes[j];
        a.expert_bytes[j] = m->expert_bytes[j];
        a.scale_offset[j] = m->scale_offset[j];
        a.k_logical[j] = m->k_logical[j];
        a.blocks_per_row[j] = m->blocks_per_row[j];
        a.n_out[j] = m->n_out[j];
    }
    a.iq2_grid = m->iq2_grid;
    a.iq2_signed = m->iq2_signed;
    a.x = d_x; a.x_pitch = x_pitch; a.y = d_y; a.y_pitch = y_pitch;
    a.logits = w->logits; a.logit_ssq = w->logit_ssq; a.ids = w->ids; a.route_weights = w->route_weights;
    a.act = w->act; a.shared_act = w->shared_act; a.shared_scale = w->shared_scale;
    a.uniq = w->uniq;
    a.ximg = w->ximg; a.aimg = w->aimg;
    a.fuse_lines = w->fuse_lines; a.fuse_gen = w->fuse_gen;
    a.error_word = w->error_word; a.exact_rows = w->exact_rows; a.route_flags = w->route_flags;
    a.x16 = w->x16; a.act16 = w->act16; a.sact16 = w->sact16;
    a.x_scale = w->x_scale; a.act_scale = w->act_scale; a.sact_scale = w->sact_scale; a.x_max2 = w->x_max2;
    a.w_norm2 = m->w_norm2; a.down = w->down;
    a.counts = w->counts; a.offsets = w->offsets; a.pair_to_row = w->pair_to_row; a.row_to_pair = w->row_to_pair;
    a.group_bad = w->group_bad; a.tiles = w->tiles;
    a.token_cap = (uint32_t)w->cap;
    a.router_t = m->router_t;
    for (int j = 0; j < 8; j++) { a.wt[j] = m->w_tiled[j]; a.wi[j] = m->w_itile[j]; a.wq[j] = m->w_qtile[j]; }
    return a;
}

struct HcTarget {   // residual streams to inject into instead of writing y
    float *residual;
    size_t token_pitch, stream_pitch;
    const float *inject;
    int streams;
};

// Most tokens the decode kernels take in one forward of this layer.
static size_t decode_limit(const PfHipMoe *moe) {
    return pf_decode_tile_layer(moe->desc, moe->w_tiled, moe->w_itile, moe->w_qtile) ? PF_TILE_DECODE_MAX_TOKENS : PF_DECODE_MAX_TOKENS;
}

static int forward_enqueue(const PfHipMoe *moe, PfHipWork *work, const float *d_x, size_t x_pitch, float *d_y,
                           size_t y_pitch, size_t tokens, const HcTarget *hc, hipStream_t s) {
    const PfHipMoeDesc *d = &moe->desc;
    if (tokens * (size_t)d->top_k > 0x7fffffffu / 4) return PF_HIP_E_UNSUPPORTED;
    PfKernelArgs a = make_args(moe, work, d_x, x_pitch, d_y, y_pitch);
    if (hc) {
        a.hc_residual = hc->residual; a.hc_inject = hc->inject; a.hc_streams = hc->streams;
        a.hc_token_pitch = hc->token_pitch; a.hc_stream_pitch = hc->stream_pitch;
    }
    if (moe->streamed) {
        snprintf(g_error, sizeof g_error, "the layer's routed experts are not resident: forward it through an expert pool");
        return PF_HIP_E_UNSUPPORTED;
    }
    const bool aligned = (x_pitch % 4 == 0) && ((uintptr_t)d_x % 16 == 0);
    if (moe->decode_ready && tokens <= decode_limit(moe) && aligned && !work->force_general) {
        pf_launch_decode(a, (int)tokens, s, work->stage_limit);
    } else if (moe->prefill_ready && work->down && tokens > PF_DECODE_MAX_TOKENS && aligned && !work->force_general) {
        pf_launch_prefill(a, (int)tokens, s, work->stage_limit);
    } else {
        // the general kernels stage one token's activations in LDS
        const size_t lds_route = ((size_t)d->hidden + 3 * (size_t)d->experts) * 4;
        if (pf_general_lds_bytes(a) > 64 * 1024 || lds_route > 64 * 1024) {
            snprintf(g_error, sizeof g_error, "dimensions exceed the LDS staging of the general kernels");
            return PF_HIP_E_UNSUPPORTED;
        }
        pf_launch_general(a, (int)tokens, s, work->stage_limit);
    }
    HIP_TRY(hipGetLastError());
    return PF_HIP_OK;
}

// Which kernels a forward of `tokens` tokens (rows 16-byte aligned) runs: 1 the decode kernels,
// 2 the matrix-core prefill kernels, 0 the general kernels.
extern "C" int pf_hip_moe_kernel_family(const PfHipMoe *moe, const PfHipWork *work, size_t tokens) {
    if (!moe || !work || work->force_general) return 0;
    if (moe->streamed) return moe->stream_decode && tokens <= PF_TILE_DECODE_MAX_TOKENS ? 1 : 0;   // given a pool with tile-ordered slots
    if (moe->decode_ready && tokens <= decode_limit(moe)) return 1;
    if (moe->prefill_ready && work->down && tokens > PF_DECODE_MAX_TOKENS) return 2;
    return 0;
}

extern "C" int pf_hip_moe_decode_launches(const PfHipMoe *moe, const PfHipWork *work, size_t tokens) {
    if (pf_hip_moe_kernel_family(moe, work, tokens) != 1 || moe->streamed) return 0;
    const PfKernelArgs a = make_args(moe, const_cast<PfHipWork *>(work), nullptr, 0, nullptr, 0);
    return pf_decode_launches(a, (int)tokens);
}

// Enqueue only: no allocation, no synchronisation, no memset; safe under stream capture.
extern "C" int pf_hip_moe_forward_device(const PfHipMoe *moe, PfHipWork *work, const float *d_x, size_t x_pitch,
                                         float *d_y, size_t y_pitch, size_t tokens, void *stream) {
    if (!moe || !work || work->moe != moe) return PF_HIP_E_ARGUMENT;
    if (tokens > work->cap) return PF_HIP_E_ARGUMENT;
    if (tokens == 0) return PF_HIP_OK;
    if (!d_x || !d_y || x_pitch < moe->desc.hidden || y_pitch < moe->desc.hidden) return PF_HIP_E_ARGUMENT;
    return forward_enqueue(moe, work, d_x, x_pitch, d_y, y_pitch, tokens, nullptr, (hipStream_t)stream);
}

// The same forward for callers that cannot allocate (code under graph capture, tight serving loops):
// the workspace is the library's static device array instead of a PfHipWork.  Calls nothing that
// allocates or frees; every call on a GPU shares that GPU's array, so calls that overlap on one GPU race.
// Nothing in the array has to start at zero: every buffer of it is written before it is read within a
// forward (the re-route counter it also holds only ever accumulates and is not reported here).
extern "C" int pf_hip_moe_forward_static(const PfHipMoe *moe, const float *d_x, size_t x_pitch, float *d_y,
                                         size_t y_pitch, uint32_t *d_ids, float *d_route_weights,
                                         uint32_t *d_error_word, size_t tokens, void *stream) {
    if (!moe || !d_error_word) return PF_HIP_E_ARGUMENT;
    if (tokens == 0) return PF_HIP_OK;
    if (!d_x || !d_y || x_pitch < moe->desc.hidden || y_pitch < moe->desc.hidden) return PF_HIP_E_ARGUMENT;
    if (tokens > PF_DECODE_MAX_TOKENS) {
        snprintf(g_error, sizeof g_error, "the static scratch serves batches of at most %d tokens, not %zu",
                 PF_DECODE_MAX_TOKENS, tokens);
        return PF_HIP_E_UNSUPPORTED;
    }
    const Carve c = plan_work(&moe->desc, tokens);
    if (c.total > PF_STATIC_SCRATCH_BYTES) {
        snprintf(g_error, sizeof g_error, "this layer needs %zu bytes of scratch for %zu tokens; the static scratch holds %zu",
                 c.total, tokens, (size_t)PF_STATIC_SCRATCH_BYTES);
        return PF_HIP_E_UNSUPPORTED;
    }
    uint8_t *base = nullptr;
    const int rc = static_scratch(&base);
    if (rc != PF_HIP_OK) return rc;
    PfHipWork w;
    memset(&w, 0, sizeof w);
    w.moe = moe; w.cap = tokens; w.bytes = c.total;
    carve_work(&w, c, base);
    if (d_ids) w.ids = d_ids;
    if (d_route_weights) w.route_weights = d_route_weights;
    w.error_word = d_error_word;
    return forward_enqueue(moe, &w, d_x, x_pitch, d_y, y_pitch, tokens, nullptr, (hipStream_t)stream);
}

// ---- hyper-connection read and add (src/qwen4_base.c:142-175) -----------------------------------
static bool hc_dims_ok(size_t tokens, size_t streams, size_t hidden) {
    return streams && hidden && tokens <= 0x7fffffffu && streams <= 0x7fffffffu && hidden <= 0x7fffffffu;
}

extern "C" int pf_hip_hc_read_device(const float *d_normed, size_t n_token_pitch, size_t n_stream_pitch,
                                     const float *d_logits, size_t g_token_pitch, size_t g_stream_pitch,
                                     float *d_mixed, size_t m_pitch, size_t tokens, size_t streams, size_t hidden,
                                     uint32_t *d_error_word, void *stream) {
    if (!hc_dims_ok(tokens, streams, hidden) || !d_error_word) return PF_HIP_E_ARGUMENT;
    if (!tokens) return PF_HIP_OK;
    if (!d_normed || !d_logits || !d_mixed || n_stream_pitch < hidden || g_stream_pitch < hidden || m_pitch < hidden)
        return PF_HIP_E_ARGUMENT;
    pf_launch_hc_read(d_normed, n_token_pitch, n_stream_pitch, d_logits, g_token_pitch, g_stream_pitch, d_mixed,
                      m_pitch, (int)tokens, (int)streams, (int)hidden, d_error_word, (hipStream_t)stream);
    HIP_TRY(hipGetLastError());
    return PF_HIP_OK;
}

extern "C" int pf_hip_hc_add_device(float *d_residual, size_t r_token_pitch, size_t r_stream_pitch,
                                    const float *d_block, size_t b_pitch, const float *d_inject, size_t i_pitch,
                                    size_t tokens, size_t streams, size_t hidden, uint32_t *d_error_word,
                                    void *stream) {
    if (!hc_dims_ok(tokens, streams, hidden) || !d_error_word) return PF_HIP_E_ARGUMENT;
    if (!tokens) return PF_HIP_OK;
    if (!d_residual || !d_block || !d_inject || r_stream_pitch < hidden || b_pitch < hidden || i_pitch < streams)
        return PF_HIP_E_ARGUMENT;
    pf_launch_hc_add(d_residual, r_token_pitch, r_stream_pitch, d_block, b_pitch, d_inject, i_pitch, (int)tokens,
                     (int)streams, (int)hidden, d_error_word, (hipStream_t)stream);
    HIP_TRY(hipGetLastError());
    return PF_HIP_OK;
}

// Enqueue only, like pf_hip_moe_forward_device: the read writes the workspace's input rows, the
// forward consumes them and its last kernel adds into the residual streams.
extern "C" int pf_hip_moe_forward_hc_device(const PfHipMoe *moe, PfHipWork *work, const float *d_normed,
                                            size_t n_token_pitch, size_t n_stream_pitch, const float *d_logits,
                                            size_t g_token_pitch, size_t g_stream_pitch, float *d_residual,
                                            size_t r_token_pitch, size_t r_stream_pitch, const float *d_inject,
                                            size_t streams, size_t tokens, void *stream) {
    if (!moe || !work || work->moe != moe || tokens > work->cap) return PF_HIP_E_ARGUMENT;
    const size_t H = moe->desc.hidden;
    if (!hc_dims_ok(tokens, streams, H)) return PF_HIP_E_ARGUMENT;
    if (!tokens) return PF_HIP_OK;
    if (!d_normed || !d_logits || !d_residual || !d_inject || n_stream_pitch < H || g_stream_pitch < H ||
        r_stream_pitch < H)
        return PF_HIP_E_ARGUMENT;
    hipStream_t s = (hipStream_t)stream;
    pf_launch_hc_read(d_normed, n_token_pitch, n_stream_pitch, d_logits, g_token_pitch, g_stream_pitch, work->x, H,
                      (int)tokens, (int)streams, (int)H, work->error_word, s);
    if (streams <= PF_HC_FOLD_MAX) {
        const HcTarget hc = {d_residual, r_token_pitch, r_stream_pitch, d_inject, (int)streams};
        return forward_enqueue(moe, work, work->x, H, work->y, H, tokens, &hc, s);
    }
    // more streams than the block's last kernel keeps in registers: the add runs as a kernel of its own
    const int rc = forward_enqueue(moe, work, work->x, H, work->y, H, tokens, nullptr, s);
    if (rc != PF_HIP_OK) return rc;
    pf_launch_hc_add(d_residual, r_token_pitch, r_stream_pitch, work->y, H, d_inject, streams, (int)tokens,
                     (int)streams, (int)H, work->error_word, s);
    HIP_TRY(hipGetLastError());
    return PF_HIP_OK;
}

extern "C" int pf_hip_moe_forward_host(const PfHipMoe *moe, PfHipWork *work, const float *x, size_t x_pitch_bytes,
                                       float *y, size_t y_pitch_bytes, uint32_t *ids, size_t ids_pitch_bytes,
                                       float *weights, size_t weights_pitch_bytes, size_t tokens,
                                       uint32_t *error_word) {
    if (!moe || !work || !error_word) return PF_HIP_E_ARGUMENT;
    *error_word = 0;
    // before any row is copied: the pinned block and the workspace's rows are sized for the workspace's own layer
    if (work->moe != moe) return PF_HIP_E_ARGUMENT;
    if (tokens == 0) return PF_HIP_OK;
    if (!x || !y || tokens > work->cap) return PF_HIP_E_ARGUMENT;
    const size_t H = moe->desc.hidden, K = moe->desc.top_k;
    if (through_host_block(work, tokens)) {
        // (the whole sequence as one replayed graph measured slower, 50 us against 43: the copies become graph nodes
        // of their own)
        const HostBlock b = host_block(&moe->desc, work->host);
        rows_in(b.x, x, x_pitch_bytes, H * 4, tokens);
        HIP_TRY(hipMemcpyAsync(work->x, b.x, tokens * H * 4, hipMemcpyHostToDevice, nullptr));
        // the last kernel writes the output rows into the pinned block itself
        int rc = pf_hip_moe_forward_device(moe, work, work->x, H, (float *)(work->host_device + b.y_offset), H, tokens, nullptr);
        if (rc != PF_HIP_OK) return rc;
        HostResults r;
        HIP_TRY(fetch_results(work, b, tokens, ids != nullptr, weights != nullptr, &r));
        HIP_TRY(hipStreamSynchronize(nullptr));
        *error_word = *r.error_word;
        if (*error_word) {
            HIP_TRY(hipMemset(work->error_word, 0, 4));   // the word is sticky on the device; reading it clears it
            return PF_HIP_OK;
        }
        rows_out(y, y_pitch_bytes, b.y, H * 4, tokens);
        if (ids) rows_out(ids, ids_pitch_bytes, r.ids, K * 4, tokens);
        if (weights) rows_out(weights, weights_pitch_bytes, r.weights, K * 4, tokens);
        return PF_HIP_OK;
    }
    HIP_TRY(hipMemcpy2D(work->x, H * 4, x, x_pitch_bytes, H * 4, tokens, hipMemcpyHostToDevice));
    // prefill-sized batches go through whole; 2..4 tokens use the decode path in one launch
    int rc = pf_hip_moe_forward_device(moe, work, work->x, H, work->y, H, tokens, nullptr);
    if (rc != PF_HIP_OK) return rc;
    HIP_TRY(hipMemcpy(error_word, work->error_word, 4, hipMemcpyDeviceToHost));
    if (*error_word) {
        HIP_TRY(hipMemset(work->error_word, 0, 4));   // the word is sticky on the device; reading it clears it
        return PF_HIP_OK;
    }
    HIP_TRY(hipMemcpy2D(y, y_pitch_bytes, work->y, H * 4, H * 4, tokens, hipMemcpyDeviceToHost));
    if (ids) HIP_TRY(hipMemcpy2D(ids, ids_pitch_bytes, work->ids, K * 4, K * 4, tokens, hipMemcpyDeviceToHost));
    if (weights)
        HIP_TRY(hipMemcpy2D(weights, weights_pitch_bytes, work->route_weights, K * 4, K * 4, tokens,
                            hipMemcpyDeviceToHost));
    return PF_HIP_OK;
}

// ---- a layer whose routed experts are streamed (src/qwen4_moe_internal.h:49-54, the remap hook) -----------------
// Two calls with the caller's pool in between.  The first runs the router and the routing and returns the pairs'
// expert ids; the caller makes those experts resident (qw4_pool_acquire) and passes the pool's device regions and
// the pairs' slots to the second, which runs the expert products and the combine reading rows at
// region + slot * expert_bytes.  The general kernels serve both: streaming is bound by the reads that fill the pool.
extern "C" int pf_hip_pool_slot_tiled(uint32_t gguf_type, size_t n_out) {
    return (gguf_type == PF_Q4_K || gguf_type == PF_IQ2_XXS) && n_out % 32 == 0;
}

// A pool region of `slots` experts of one matrix in the layout the kernels read a slot in: pf_tensor_place (a resident
// tensor of `slots` experts; Q4_K tile order has the file's size), or for IQ2_XXS slots in tile order the chunks of
// pf_decode_addr.h with the block scales inside them.
struct SlotPlan { size_t region_bytes, file_expert_bytes, expert_bytes, scale_offset; int blocks_per_row; };
static bool slot_plan(uint32_t gguf_type, size_t k_storage, size_t n_out, size_t slots, SlotPlan *p) {
    PfTensorPlace place;
    if (!slots || !n_out || !pf_tensor_place(gguf_type, k_storage, n_out, slots, &place)) return false;
    p->region_bytes = place.bytes;
    p->file_expert_bytes = place.gguf_bytes / slots;
    p->expert_bytes = place.expert_bytes;
    p->scale_offset = place.scale_offset;
    p->blocks_per_row = place.blocks_per_row;
    if (gguf_type == PF_IQ2_XXS && pf_hip_pool_slot_tiled(gguf_type, n_out)) {
        p->expert_bytes = pf_i2t_expert_bytes((int)n_out, place.blocks_per_row);
        p->region_bytes = p->expert_bytes * slots;
        p->scale_offset = 0;
    }
    return true;
}

// Short batches of a streamed layer whose Q4_K pool regions hold tile-ordered slots (all three of a Q4_K layer; gate and
// up of the q4 checkpoint profile, whose MXFP4 down slots stay row by row) run the tile decode kernels: kernel 1 and the
// routing kernels in the first call, kernels 2 and 3 reading the pairs' slots in the second.
static bool streamed_decode(const PfHipMoe *moe, const PfHipWork *work, size_t tokens, uint32_t tiled_mask) {
    const uint32_t wanted = moe->stream_decode <= 2 ? 7u : 3u;   // one format throughout: all three regions; a profile: gate and up
    return moe->stream_decode && tiled_mask == wanted && tokens <= PF_TILE_DECODE_MAX_TOKENS && !work->force_general;
}

extern "C" int pf_hip_moe_route_streamed_host(const PfHipMoe *moe, PfHipWork *work, const float *x, size_t x_pitch_bytes,
                                              size_t tokens, uint32_t tiled_mask, uint32_t *ids, uint32_t *error_word) {
    if (!moe || !work || work->moe != moe || !error_word) return PF_HIP_E_ARGUMENT;
    *error_word = 0;
    if (tokens == 0) return PF_HIP_OK;
    if (!x || !ids || tokens > work->cap) return PF_HIP_E_ARGUMENT;
    const size_t H = moe->desc.hidden, K = moe->desc.top_k;
    if (tokens * K > 0x7fffffffu / 4) return PF_HIP_E_UNSUPPORTED;
    const bool staged = through_host_block(work, tokens);
    const HostBlock b = host_block(&moe->desc, work->host);
    if (staged) {
        rows_in(b.x, x, x_pitch_bytes, H * 4, tokens);
        HIP_TRY(hipMemcpyAsync(work->x, b.x, tokens * H * 4, hipMemcpyHostToDevice, nullptr));
    } else {
        HIP_TRY(hipMemcpy2D(work->x, H * 4, x, x_pitch_bytes, H * 4, tokens, hipMemcpyHostToDevice));
    }
    PfKernelArgs a = make_args(moe, work, work->x, H, work->y, H);
    const size_t lds_route = (H + 3 * (size_t)moe->desc.experts) * 4;
    if (pf_general_lds_bytes(a) > 64 * 1024 || lds_route > 64 * 1024) {
        snprintf(g_error, sizeof g_error, "dimensions exceed the LDS staging of the general kernels");
        return PF_HIP_E_UNSUPPORTED;
    }
    if (streamed_decode(moe, work, tokens, tiled_mask)) {
        HIP_TRY(hipMemsetAsync(work->route_flags, 0, 4, nullptr));   // the routing's list starts empty (the other router kernels clear it themselves)
        pf_launch_dec_router(a, (int)tokens, (int)((moe->desc.experts + 3) / 4), nullptr);
        pf_launch_route(a, (int)tokens, nullptr);
    } else {
        pf_launch_general(a, (int)tokens, nullptr, 2);
    }
    HIP_TRY(hipGetLastError());
    HostResults r = {nullptr, nullptr, nullptr};
    if (staged) {
        HIP_TRY(fetch_results(work, b, tokens, true, false, &r));
        HIP_TRY(hipStreamSynchronize(nullptr));
        *error_word = *r.error_word;
    } else {
        HIP_TRY(hipMemcpy(error_word, work->error_word, 4, hipMemcpyDeviceToHost));
    }
    if (*error_word) {
        HIP_TRY(hipMemset(work->error_word, 0, 4));
        return PF_HIP_OK;
    }
    if (staged) memcpy(ids, r.ids, tokens * K * 4);
    else HIP_TRY(hipMemcpy(ids, work->ids, tokens * K * 4, hipMemcpyDeviceToHost));
    return PF_HIP_OK;
}

extern "C" int pf_hip_moe_experts_streamed_host(const PfHipMoe *moe, PfHipWork *work, const void *const regions[3],
                                                const size_t expert_bytes[3], const size_t scale_offsets[3],
                                                uint32_t pool_slots, uint32_t tiled_mask, const uint32_t *slots,
                                                float *y, size_t y_pitch_bytes, uint32_t *ids, size_t ids_pitch_bytes,
                                                float *weights, size_t weights_pitch_bytes, size_t tokens,
                                                uint32_t *error_word) {
    if (!moe || !work || work->moe != moe || !error_word || !regions || !expert_bytes) return PF_HIP_E_ARGUMENT;
    *error_word = 0;
    if (tokens == 0) return PF_HIP_OK;
    if (!y || !slots || !pool_slots || tokens > work->cap) return PF_HIP_E_ARGUMENT;
    const size_t H = moe->desc.hidden, K = moe->desc.top_k;
    for (int j = 0; j < 3; j++) {   // a slot holds one expert of each tensor in the device layout of `pool_slots` experts
        PfTensorPlace place;
        SlotPlan plan;
        const int t = 1 + j;
        const size_t k_storage = t == 3 ? moe->desc.down_physical : moe->desc.hidden;
        if (!regions[j] || !scale_offsets || !pf_tensor_place(moe->desc.type[t], k_storage, (size_t)moe->n_out[t], pool_slots, &place) ||
            !slot_plan(moe->desc.type[t], k_storage, (size_t)moe->n_out[t], pool_slots, &plan))
            return PF_HIP_E_ARGUMENT;
        const bool tiled = (tiled_mask >> j) & 1u;   // a pool of file bytes under split formats is refused further down
        const size_t want_bytes = tiled ? plan.expert_bytes : place.expert_bytes, want_scales = tiled ? plan.scale_offset : place.scale_offset;
        if (expert_bytes[j] != want_bytes || scale_offsets[j] != want_scales) return PF_HIP_E_ARGUMENT;
    }
    const bool staged = through_host_block(work, tokens);
    const HostBlock b = host_block(&moe->desc, work->host);
    if (staged) {
        memcpy(b.slots, slots, tokens * K * 4);
        HIP_TRY(hipMemcpyAsync(work->slots, b.slots, tokens * K * 4, hipMemcpyHostToDevice, nullptr));
    } else {
        HIP_TRY(hipMemcpy(work->slots, slots, tokens * K * 4, hipMemcpyHostToDevice));
    }
    PfKernelArgs a = make_args(moe, work, work->x, H, staged ? (float *)(work->host_device + b.y_offset) : work->y, H);
    for (int j = 0; j < 3; j++) {
        const int t = 1 + j;
        const bool tiled = (tiled_mask >> j) & 1u;
        if (tiled && !pf_hip_pool_slot_tiled(moe->desc.type[t], (size_t)moe->n_out[t])) return PF_HIP_E_ARGUMENT;
        const bool iq2 = moe->desc.type[t] == PF_IQ2_XXS;
        a.w[t] = tiled ? nullptr : static_cast<const uint8_t *>(regions[j]);    // slots in tile order: every kernel's tile reader
        a.wt[t] = tiled && !iq2 ? static_cast<const uint8_t *>(regions[j]) : nullptr;
        a.wi[t] = tiled && iq2 ? static_cast<const uint8_t *>(regions[j]) : nullptr;
        a.scale_offset[t] = scale_offsets[j];
    }
    a.slots = work->slots;
    a.pool_slots = pool_slots;
    if (streamed_decode(moe, work, tokens, tiled_mask)) {
        // kernel 1 ran in the first call (logits and the token rows' images are in the workspace): kernels 2 and 3 only
        pf_launch_decode_stream_experts(a, (int)tokens, nullptr);
    } else {
        pf_launch_general(a, (int)tokens, nullptr, 0, 3);
    }
    HIP_TRY(hipGetLastError());
    if (staged) {
        HostResults r;
        HIP_TRY(fetch_results(work, b, tokens, ids != nullptr, weights != nullptr, &r));
        HIP_TRY(hipStreamSynchronize(nullptr));
        *error_word = *r.error_word;
        if (*error_word) {
            HIP_TRY(hipMemset(work->error_word, 0, 4));
            return PF_HIP_OK;
        }
        rows_out(y, y_pitch_bytes, b.y, H * 4, tokens);
        if (ids) rows_out(ids, ids_pitch_bytes, r.ids, K * 4, tokens);
        if (weights) rows_out(weights, weights_pitch_bytes, r.weights, K * 4, tokens);
        return PF_HIP_OK;
    }
    HIP_TRY(hipMemcpy(error_word, work->error_word, 4, hipMemcpyDeviceToHost));
    if (*error_word) {
        HIP_TRY(hipMemset(work->error_word, 0, 4));
        return PF_HIP_OK;
    }
    HIP_TRY(hipMemcpy2D(y, y_pitch_bytes, work->y, H * 4, H * 4, tokens, hipMemcpyDeviceToHost));
    if (ids) HIP_TRY(hipMemcpy2D(ids, ids_pitch_bytes, work->ids, K * 4, K * 4, tokens, hipMemcpyDeviceToHost));
    if (weights)
        HIP_TRY(hipMemcpy2D(weights, weights_pitch_bytes, work->route_weights, K * 4, K * 4, tokens,
                            hipMemcpyDeviceToHost));
    return PF_HIP_OK;
}

struct DeviceBlock {   // one allocation, freed on scope exit
    uint8_t *p = nullptr;
    ~DeviceBlock() { if (p) (void)hipFree(p); }
};

// Pool slots in the device layout (the pool itself is C11 and knows no layouts).  A region holds `slots` experts of one
// matrix exactly as a resident tensor of `slots` experts would be laid out (pf_tensor_place): formats stored as the file
// stores them slot after slot; formats stored split as all payloads, then (256-aligned) all scales.
extern "C" int pf_hip_pool_region_plan(uint32_t gguf_type, size_t k_storage, size_t n_out, size_t slots, size_t *region_bytes,
                                       size_t *file_expert_bytes, size_t *payload_expert_bytes, size_t *scale_offset) {
    SlotPlan plan;
    if (!region_bytes || !file_expert_bytes || !payload_expert_bytes || !scale_offset ||
        !slot_plan(gguf_type, k_storage, n_out, slots, &plan))
        return PF_HIP_E_ARGUMENT;
    *region_bytes = plan.region_bytes;
    *file_expert_bytes = plan.file_expert_bytes;
    *payload_expert_bytes = plan.expert_bytes;
    *scale_offset = plan.scale_offset;
    return PF_HIP_OK;
}

// ---- a reader's staging (expert streaming): page-locked host memory the file is read into, device memory the bytes are
// copied to before a split or tile kernel lays them out in the slot, and a stream of the reader's own, all allocated once
struct PfHipStage {
    uint8_t *host, *device;
    uint8_t *split;   // the split form of an IQ2_XXS matrix on its way into the tile order (bytes + 256)
    size_t bytes;
    hipStream_t stream;
};

extern "C" int pf_hip_stage_create(size_t bytes, PfHipStage **out) {
    if (!out || !bytes) return PF_HIP_E_ARGUMENT;
    *out = nullptr;
    PfHipStage *st = (PfHipStage *)calloc(1, sizeof *st);
    if (!st) return PF_HIP_E_MEMORY;
    st->bytes = bytes;
    hipError_t e = hipHostMalloc((void **)&st->host, bytes, hipHostMallocDefault);
    if (e == hipSuccess) e = hipMalloc((void **)&st->device, bytes);
    if (e == hipSuccess) e = hipMalloc((void **)&st->split, bytes + 256);
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&st->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
        pf_set_error("staging of an expert pool's reader", e);
        if (st->host) (void)hipHostFree(st->host);
        if (st->device) (void)hipFree(st->device);
        if (st->split) (void)hipFree(st->split);
        free(st);
        return PF_HIP_E_MEMORY;
    }
    *out = st;
    return PF_HIP_OK;
}

extern "C" void pf_hip_stage_destroy(PfHipStage *st) {
    if (!st) return;
    (void)hipStreamDestroy(st->stream);
    (void)hipHostFree(st->host);
    (void)hipFree(st->device);
    (void)hipFree(st->split);
    free(st);
}

extern "C" void *pf_hip_stage_host(PfHipStage *st) { return st ? st->host : nullptr; }

// The expert the stage's host memory holds (one expert's slice of one matrix, as the file stores it) into slot `slot` of
// the matrix's region: gguf_type == UINT32_MAX copies `file_bytes` bytes as they are to region + slot * file_bytes.
// Enqueued on the stage's stream and waited for: no allocation, and readers with stages of their own run side by side.
extern "C" int pf_hip_pool_store_staged(PfHipStage *st, uint32_t gguf_type, size_t k_storage, size_t n_out, size_t slots, void *region,
                                        size_t slot, size_t file_bytes) {
    if (!st || !region || slot >= slots || file_bytes > st->bytes) return PF_HIP_E_ARGUMENT;
    uint8_t *base = static_cast<uint8_t *>(region);
    if (gguf_type == UINT32_MAX) {
        HIP_TRY(hipMemcpyAsync(base + slot * file_bytes, st->host, file_bytes, hipMemcpyHostToDevice, st->stream));
        HIP_TRY(hipStreamSynchronize(st->stream));
        return PF_HIP_OK;
    }
    PfTensorPlace place;
    SlotPlan plan;
    if (!pf_tensor_place(gguf_type, k_storage, n_out, slots, &place) || !slot_plan(gguf_type, k_storage, n_out, slots, &plan) ||
        plan.file_expert_bytes != file_bytes)
        return PF_HIP_E_ARGUMENT;
    const size_t head = split_header_bytes(gguf_type);
    if (!pf_hip_pool_slot_tiled(gguf_type, n_out) && !head) {   // as the file stores it
        HIP_TRY(hipMemcpyAsync(base + slot * place.expert_bytes, st->host, file_bytes, hipMemcpyHostToDevice, st->stream));
        HIP_TRY(hipStreamSynchronize(st->stream));
        return PF_HIP_OK;
    }
    HIP_TRY(hipMemcpyAsync(st->device, st->host, file_bytes, hipMemcpyHostToDevice, st->stream));
    if (pf_hip_pool_slot_tiled(gguf_type, n_out) && gguf_type == PF_IQ2_XXS) {
        // payloads and scales apart (the upload's split kernel, into the stage), then into the slot in tile order
        PfTensorPlace one;
        if (!pf_tensor_place(gguf_type, k_storage, n_out, 1, &one) || one.bytes > st->bytes + 256) return PF_HIP_E_ARGUMENT;
        const size_t blocks = (size_t)one.blocks_per_row * n_out;
        pf_launch_iq2_split(st->device, st->split, reinterpret_cast<uint16_t *>(st->split + one.scale_offset), blocks, st->stream);
        pf_launch_iq2_tile(st->split, reinterpret_cast<const uint16_t *>(st->split + one.scale_offset), base + slot * plan.expert_bytes,
                           n_out, one.blocks_per_row, st->stream);
    } else if (pf_hip_pool_slot_tiled(gguf_type, n_out)) {   // Q4_K: the slot in the tile order every kernel family reads
        pf_launch_q4k_tile(st->device, base + slot * place.expert_bytes, n_out, place.blocks_per_row, st->stream);
    } else {
        size_t block, size;
        block_geometry(gguf_type, &block, &size);
        const size_t blocks = (size_t)place.blocks_per_row * n_out;
        uint8_t *payload = base + slot * place.expert_bytes, *scales = base + place.scale_offset + slot * blocks * head;
        if (gguf_type == PF_IQ2_XXS) pf_launch_iq2_split(st->device, payload, reinterpret_cast<uint16_t *>(scales), blocks, st->stream);
        else pf_launch_block_split(st->device, payload, scales, blocks, (int)size, (int)head, st->stream);
    }
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipStreamSynchronize(st->stream));
    return PF_HIP_OK;
}

// One expert's slice of one matrix, as the file stores it, into slot `slot` of the matrix's region.
extern "C" int pf_hip_pool_store(uint32_t gguf_type, size_t k_storage, size_t n_out, size_t slots, void *region, size_t slot,
                                 const void *file_bytes) {
    PfTensorPlace place;
    if (!region || !file_bytes || slot >= slots || !pf_tensor_place(gguf_type, k_storage, n_out, slots, &place))
        return PF_HIP_E_ARGUMENT;
    uint8_t *base = static_cast<uint8_t *>(region);
    const size_t head = split_header_bytes(gguf_type), file_expert = place.gguf_bytes / slots;
    if (pf_hip_pool_slot_tiled(gguf_type, n_out) && gguf_type == PF_IQ2_XXS) {
        PfTensorPlace one;
        SlotPlan plan;
        if (!pf_tensor_place(gguf_type, k_storage, n_out, 1, &one) || !slot_plan(gguf_type, k_storage, n_out, slots, &plan)) return PF_HIP_E_ARGUMENT;
        DeviceBlock staging, split;
        HIP_TRY(hipMalloc((void **)&staging.p, file_expert));
        HIP_TRY(hipMalloc((void **)&split.p, one.bytes));
        HIP_TRY(hipMemcpy(staging.p, file_bytes, file_expert, hipMemcpyHostToDevice));
        const size_t blocks = (size_t)one.blocks_per_row * n_out;
        pf_launch_iq2_split(staging.p, split.p, reinterpret_cast<uint16_t *>(split.p + one.scale_offset), blocks, nullptr);
        pf_launch_iq2_tile(split.p, reinterpret_cast<const uint16_t *>(split.p + one.scale_offset), base + slot * plan.expert_bytes, n_out,
                           one.blocks_per_row, nullptr);
        HIP_TRY(hipGetLastError());
        HIP_TRY(hipStreamSynchronize(nullptr));
        return PF_HIP_OK;
    }
    if (pf_hip_pool_slot_tiled(gguf_type, n_out)) {   // Q4_K: the slot in the tile order every kernel family reads
        DeviceBlock staging;
        HIP_TRY(hipMalloc((void **)&staging.p, file_expert));
        HIP_TRY(hipMemcpy(staging.p, file_bytes, file_expert, hipMemcpyHostToDevice));
        pf_launch_q4k_tile(staging.p, base + slot * place.expert_bytes, n_out, place.blocks_per_row, nullptr);
        HIP_TRY(hipGetLastError());
        HIP_TRY(hipStreamSynchronize(nullptr));
        return PF_HIP_OK;
    }
    if (!head) {
        HIP_TRY(hipMemcpy(base + slot * place.expert_bytes, file_bytes, file_expert, hipMemcpyHostToDevice));
        return PF_HIP_OK;
    }
    size_t block, size;
    block_geometry(gguf_type, &block, &size);
    DeviceBlock staging;
    HIP_TRY(hipMalloc((void **)&staging.p, file_expert));
    HIP_TRY(hipMemcpy(staging.p, file_bytes, file_expert, hipMemcpyHostToDevice));
    const size_t blocks = (size_t)place.blocks_per_row * n_out;
    uint8_t *payload = base + slot * place.expert_bytes, *scales = base + place.scale_offset + slot * blocks * head;
    if (gguf_type == PF_IQ2_XXS) pf_launch_iq2_split(staging.p, payload, reinterpret_cast<uint16_t *>(scales), blocks, nullptr);
    else pf_launch_block_split(staging.p, payload, scales, blocks, (int)size, (int)head, nullptr);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipStreamSynchronize(nullptr));
    return PF_HIP_OK;
}

// ---- stand-alone operators on host buffers ---------------------------------------

// A [tokens, streams, hidden] cube between host memory (byte pitches) and a dense device array.
static hipError_t copy_cube(void *dense, void *host, size_t token_pitch, size_t stream_pitch, size_t T, size_t S,
                            size_t H, bool to_device) {
    const size_t row = H * 4;
    const hipMemcpyKind kind = to_device ? hipMemcpyHostToDevice : hipMemcpyDeviceToHost;
    if (T == 1 || S == 1 || token_pitch == S * stream_pitch) {   // one pitch describes every row
        const size_t pitch = S == 1 ? token_pitch : stream_pitch;
        return to_device ? hipMemcpy2D(dense, row, host, pitch, row, T * S, kind)
                         : hipMemcpy2D(host, pitch, dense, row, row, T * S, kind);
    }
    for (size_t t = 0; t < T; t++) {
        uint8_t *h = (uint8_t *)host + t * token_pitch, *d = (uint8_t *)dense + t * S * row;
        const hipError_t e = to_device ? hipMemcpy2D(d, row, h, stream_pitch, row, S, kind)
                                       : hipMemcpy2D(h, stream_pitch, d, row, row, S, kind);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}
static size_t pad256(size_t n) { return (n + 255) & ~(size_t)255; }

extern "C" int pf_hip_hc_read_host(const float *normed, size_t n_token_pitch_bytes, size_t n_stream_pitch_bytes,
                                   const float *logits, size_t g_token_pitch_bytes, size_t g_stream_pitch_bytes,
                                   float *mixed, size_t m_pitch_bytes, size_t tokens, size_t streams, size_t hidden,
                                   uint32_t *error_word) {
    if (!error_word) return PF_HIP_E_ARGUMENT;
    *error_word = 0;
    if (!hc_dims_ok(tokens, streams, hidden)) return PF_HIP_E_ARGUMENT;
    if (!tokens) return PF_HIP_OK;
    if (!normed || !logits || !mixed) return PF_HIP_E_ARGUMENT;
    if (need_device()) return PF_HIP_E_NO_DEVICE;
    const size_t cube = pad256(tokens * streams * hidden * 4), out = pad256(tokens * hidden * 4);
    DeviceBlock blk;
    HIP_TRY(hipMalloc((void **)&blk.p, 2 * cube + out + 256));
    float *d_n = (float *)blk.p, *d_g = (float *)(blk.p + cube), *d_m = (float *)(blk.p + 2 * cube);
    uint32_t *d_err = (uint32_t *)(blk.p + 2 * cube + out);
    HIP_TRY(copy_cube(d_n, (void *)normed, n_token_pitch_bytes, n_stream_pitch_bytes, tokens, streams, hidden, true));
    HIP_TRY(copy_cube(d_g, (void *)logits, g_token_pitch_bytes, g_stream_pitch_bytes, tokens, streams, hidden, true));
    HIP_TRY(hipMemset(d_err, 0, 256));
    pf_launch_hc_read(d_n, streams * hidden, hidden, d_g, streams * hidden, hidden, d_m, hidden, (int)tokens,
                      (int)streams, (int)hidden, d_err, nullptr);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipMemcpy(error_word, d_err, 4, hipMemcpyDeviceToHost));
    if (*error_word) return PF_HIP_OK;
    HIP_TRY(hipMemcpy2D(mixed, m_pitch_bytes, d_m, hidden * 4, hidden * 4, tokens, hipMemcpyDeviceToHost));
    return PF_HIP_OK;
}

extern "C" int pf_hip_hc_add_host(float *residual, size_t r_token_pitch_bytes, size_t r_stream_pitch_bytes,
                                  const float *block, size_t b_pitch_bytes, const float *inject,
                                  size_t i_pitch_bytes, size_t tokens, size_t streams, size_t hidden,
                                  uint32_t *error_word) {
    if (!error_word) return PF_HIP_E_ARGUMENT;
    *error_word = 0;
    if (!hc_dims_ok(tokens, streams, hidden)) return PF_HIP_E_ARGUMENT;
    if (!tokens) return PF_HIP_OK;
    if (!residual || !block || !inject) return PF_HIP_E_ARGUMENT;
    if (need_device()) return PF_HIP_E_NO_DEVICE;
    const size_t cube = pad256(tokens * streams * hidden * 4), rows = pad256(tokens * hidden * 4),
                 gates = pad256(tokens * streams * 4);
    DeviceBlock blk;
    HIP_TRY(hipMalloc((void **)&blk.p, cube + rows + gates + 256));
    float *d_r = (float *)blk.p, *d_b = (float *)(blk.p + cube), *d_i = (float *)(blk.p + cube + rows);
    uint32_t *d_err = (uint32_t *)(blk.p + cube + rows + gates);
    HIP_TRY(copy_cube(d_r, residual, r_token_pitch_bytes, r_stream_pitch_bytes, tokens, streams, hidden, true));
    HIP_TRY(hipMemcpy2D(d_b, hidden * 4, block, b_pitch_bytes, hidden * 4, tokens, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy2D(d_i, streams * 4, inject, i_pitch_bytes, streams * 4, tokens, hipMemcpyHostToDevice));
    HIP_TRY(hipMemset(d_err, 0, 256));
    pf_launch_hc_add(d_r, streams * hidden, hidden, d_b, hidden, d_i, streams, (int)tokens, (int)streams, (int)hidden,
                     d_err, nullptr);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipMemcpy(error_word, d_err, 4, hipMemcpyDeviceToHost));
    if (*error_word) return PF_HIP_OK;
    HIP_TRY(copy_cube(d_r, residual, r_token_pitch_bytes, r_stream_pitch_bytes, tokens, streams, hidden, false));
    return PF_HIP_OK;
}

extern "C" int pf_hip_moe_forward_hc_host(const PfHipMoe *moe, PfHipWork *work, const float *normed,
                                          size_t n_token_pitch_bytes, size_t n_stream_pitch_bytes,
                                          const float *logits, size_t g_token_pitch_bytes,
                                          size_t g_stream_pitch_bytes, float *residual, size_t r_token_pitch_bytes,
                                          size_t r_stream_pitch_bytes, const float *inject, size_t i_pitch_bytes,
                                          size_t streams, size_t tokens, uint32_t *ids, size_t ids_pitch_bytes,
                                          float *weights, size_t weights_pitch_bytes, uint32_t *error_word) {
    if (!moe || !work || !error_word) return PF_HIP_E_ARGUMENT;
    *error_word = 0;
    const size_t H = moe->desc.hidden, K = moe->desc.top_k;
    if (!hc_dims_ok(tokens, streams, H) || tokens > work->cap) return PF_HIP_E_ARGUMENT;
    if (!tokens) return PF_HIP_OK;
    if (!normed || !logits || !residual || !inject) return PF_HIP_E_ARGUMENT;
    const size_t cube = pad256(tokens * streams * H * 4), gates = pad256(tokens * streams * 4);
    DeviceBlock blk;
    HIP_TRY(hipMalloc((void **)&blk.p, 3 * cube + gates));
    float *d_n = (float *)blk.p, *d_g = (float *)(blk.p + cube), *d_r = (float *)(blk.p + 2 * cube),
          *d_i = (float *)(blk.p + 3 * cube);
    HIP_TRY(copy_cube(d_n, (void *)normed, n_token_pitch_bytes, n_stream_pitch_bytes, tokens, streams, H, true));
    HIP_TRY(copy_cube(d_g, (void *)logits, g_token_pitch_bytes, g_stream_pitch_bytes, tokens, streams, H, true));
    HIP_TRY(copy_cube(d_r, residual, r_token_pitch_bytes, r_stream_pitch_bytes, tokens, streams, H, true));
    HIP_TRY(hipMemcpy2D(d_i, streams * 4, inject, i_pitch_bytes, streams * 4, tokens, hipMemcpyHostToDevice));
    int rc = pf_hip_moe_forward_hc_device(moe, work, d_n, streams * H, H, d_g, streams * H, H, d_r, streams * H, H,
                                          d_i, streams, tokens, nullptr);
    if (rc != PF_HIP_OK) return rc;
    HIP_TRY(hipMemcpy(error_word, work->error_word, 4, hipMemcpyDeviceToHost));
    if (*error_word) {
        HIP_TRY(hipMemset(work->error_word, 0, 4));   // the word is sticky on the device; reading it clears it
        return PF_HIP_OK;
    }
    HIP_TRY(copy_cube(d_r, residual, r_token_pitch_bytes, r_stream_pitch_bytes, tokens, streams, H, false));
    if (ids) HIP_TRY(hipMemcpy2D(ids, ids_pitch_bytes, work->ids, K * 4, K * 4, tokens, hipMemcpyDeviceToHost));
    if (weights)
        HIP_TRY(hipMemcpy2D(weights, weights_pitch_bytes, work->route_weights, K * 4, K * 4, tokens,
                            hipMemcpyDeviceToHost));
    return PF_HIP_OK;
}

extern "C" int pf_hip_route_host(const float *logits, size_t tokens, size_t experts, size_t top_k, int norm_topk,
                                 float *probs, uint32_t *ids, float *weights, uint32_t *error_word,
                                 uint64_t *bad_row) {
    if (!error_word) return PF_HIP_E_ARGUMENT;
    *error_word = 0;
    if (bad_row) *bad_row = 0;
    if (tokens == 0) return PF_HIP_OK;
    if (!logits || !probs || !ids || !weights || !experts || !top_k || top_k > experts) return PF_HIP_E_ARGUMENT;
    if (tokens * experts > 0x7fffffffu) return PF_HIP_E_UNSUPPORTED;
    if (need_device()) return PF_HIP_E_NO_DEVICE;
    const size_t zb = tokens * experts * 4, kb = tokens * top_k * 4;
    const size_t o_p = (zb + 255) & ~(size_t)255, o_i = o_p * 2, o_w = o_i + ((kb + 255) & ~(size_t)255),
                 o_e = o_w + ((kb + 255) & ~(size_t)255);
    DeviceBlock blk;
    HIP_TRY(hipMalloc((void **)&blk.p, o_e + 256));
    HIP_TRY(hipMemcpy(blk.p, logits, zb, hipMemcpyHostToDevice));
    unsigned long long init[2] = {0ull, ~0ull};   // error word, first bad row
    HIP_TRY(hipMemcpy(blk.p + o_e, init, sizeof init, hipMemcpyHostToDevice));
    int rc = pf_route_exact_device((const float *)blk.p, (int)tokens, (int)experts, (int)top_k, norm_topk,
                                   (float *)(blk.p + o_p), (uint32_t *)(blk.p + o_i), (float *)(blk.p + o_w),
                                   (uint32_t *)(blk.p + o_e), (unsigned long long *)(blk.p + o_e + 8), nullptr);
    if (rc != PF_HIP_OK) return rc;
    HIP_TRY(hipDeviceSynchronize());
    unsigned long long back[2];
    HIP_TRY(hipMemcpy(back, blk.p + o_e, sizeof back, hipMemcpyDeviceToHost));
    *error_word = (uint32_t)back[0];
    if (*error_word) {
        if (bad_row) *bad_row = back[1];
        return PF_HIP_OK;
    }
    HIP_TRY(hipMemcpy(probs, blk.p + o_p, zb, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(ids, blk.p + o_i, kb, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(weights, blk.p + o_w, kb, hipMemcpyDeviceToHost));
    return PF_HIP_OK;
}

extern "C" int pf_hip_group_pairs_host(const uint32_t *ids, size_t tokens, size_t experts, size_t top_k,
                                       uint64_t *offsets, uint64_t *pair_to_row, uint64_t *row_to_pair,
                                       uint32_t *error_word, int *duplicate) {
    if (!error_word || !duplicate || !offsets || !experts || !top_k) return PF_HIP_E_ARGUMENT;
    *error_word = 0;
    *duplicate = 0;
    const size_t pairs = tokens * top_k;
    if (pairs > 0x3fffffffu || experts > 0x3fffffffu) return PF_HIP_E_UNSUPPORTED;
    if (need_device()) return PF_HIP_E_NO_DEVICE;
    if (pairs && (!ids || !pair_to_row || !row_to_pair)) return PF_HIP_E_ARGUMENT;
    const size_t pb = ((pairs ? pairs : 1) * 4 + 255) & ~(size_t)255, eb = ((experts + 1) * 4 + 255) & ~(size_t)255;
    // ids | counts | offsets | pair_to_row | row_to_pair | first offending pair
    DeviceBlock blk;
    HIP_TRY(hipMalloc((void **)&blk.p, 3 * pb + 2 * eb + 256));
    uint32_t *d_ids = (uint32_t *)blk.p, *d_counts = (uint32_t *)(blk.p + pb), *d_off = (uint32_t *)(blk.p + pb + eb);
    uint32_t *d_p2r = (uint32_t *)(blk.p + pb + 2 * eb), *d_r2p = (uint32_t *)(blk.p + 2 * pb + 2 * eb);
    uint32_t *d_bad = (uint32_t *)(blk.p + 3 * pb + 2 * eb);
    if (pairs) HIP_TRY(hipMemcpy(d_ids, ids, pairs * 4, hipMemcpyHostToDevice));
    int rc = pf_group_pairs_device(d_ids, (int)tokens, (int)experts, (int)top_k, d_counts, d_off, d_p2r, d_r2p, d_bad,
                                   nullptr);
    if (rc != PF_HIP_OK) return rc;
    HIP_TRY(hipDeviceSynchronize());
    uint32_t bad = 0;
    HIP_TRY(hipMemcpy(&bad, d_bad, 4, hipMemcpyDeviceToHost));
    if (bad != 0xffffffffu) {   // first offending pair in scan order, low bit = kind
        if (bad & 1u) *duplicate = 1;
        else *error_word = PF_HIP_ERR_BOUNDS;
        return PF_HIP_OK;
    }
    uint32_t *host = (uint32_t *)malloc(((experts + 1) > pairs ? (experts + 1) : pairs) * 4);
    if (!host) return PF_HIP_E_MEMORY;
    hipError_t e = hipMemcpy(host, d_off, (experts + 1) * 4, hipMemcpyDeviceToHost);
    for (size_t j = 0; e == hipSuccess && j <= experts; j++) offsets[j] = host[j];
    if (e == hipSuccess && pairs) {
        e = hipMemcpy(host, d_p2r, pairs * 4, hipMemcpyDeviceToHost);
        for (size_t j = 0; e == hipSuccess && j < pairs; j++) pair_to_row[j] = host[j];
        if (e == hipSuccess) e = hipMemcpy(host, d_r2p, pairs * 4, hipMemcpyDeviceToHost);
        for (size_t j = 0; e == hipSuccess && j < pairs; j++) row_to_pair[j] = host[j];
    }
    free(host);
    if (e != hipSuccess) { pf_set_error("group download", e); return PF_HIP_E_RUNTIME; }
    return PF_HIP_OK;
}

extern "C" int pf_hip_packed_matmul_host(uint32_t gguf_type, const void *expert_bytes, size_t row_bytes, size_t n_out,
                                         size_t k_logical, const float *x, size_t rows, float *y,
                                         uint32_t *error_word) {
    if (!error_word) return PF_HIP_E_ARGUMENT;
    *error_word = 0;
    if (rows == 0) return PF_HIP_OK;
    size_t block, size;
    if (!block_geometry(gguf_type, &block, &size)) return PF_HIP_E_UNSUPPORTED;
    if (!expert_bytes || !x || !y || !n_out || !k_logical) return PF_HIP_E_ARGUMENT;
    if (rows * n_out > 0x7fffffffu || k_logical > 0x7fffffffu) return PF_HIP_E_UNSUPPORTED;
    if (need_device()) return PF_HIP_E_NO_DEVICE;
    const uint64_t *grid = pf_device_iq2_grid();
    if (!grid) return PF_HIP_E_MEMORY;
    const size_t wb = (row_bytes * n_out + 255) & ~(size_t)255, xb = (rows * k_logical * 4 + 255) & ~(size_t)255,
                 yb = (rows * n_out * 4 + 255) & ~(size_t)255;
    DeviceBlock blk;
    HIP_TRY(hipMalloc((void **)&blk.p, wb + xb + yb + 256));
    HIP_TRY(upload_from_host(blk.p, expert_bytes, row_bytes * n_out));
    HIP_TRY(hipMemcpy(blk.p + wb, x, rows * k_logical * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemset(blk.p + wb + xb + yb, 0, 256));
    pf_launch_exact_matmul(gguf_type, blk.p, row_bytes, (int)n_out, (int)k_logical, (const float *)(blk.p + wb),
                           (int)rows, (float *)(blk.p + wb + xb), (uint32_t *)(blk.p + wb + xb + yb), grid, nullptr);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipMemcpy(error_word, blk.p + wb + xb + yb, 4, hipMemcpyDeviceToHost));
    if (*error_word) return PF_HIP_OK;
    HIP_TRY(hipMemcpy(y, blk.p + wb + xb, rows * n_out * 4, hipMemcpyDeviceToHost));
    return PF_HIP_OK;
}

extern "C" int pf_hip_exact_elementwise_host(int op, const float *a, const float *b, size_t n, float *out,
                                            uint32_t *error_word) {
    if (!error_word) return PF_HIP_E_ARGUMENT;
    *error_word = 0;
    if (op < 0 || op > 2) return PF_HIP_E_UNSUPPORTED;
    if (n == 0) return PF_HIP_OK;
    if (!a || !out || (op == 2 && !b)) return PF_HIP_E_ARGUMENT;
    if (need_device()) return PF_HIP_E_NO_DEVICE;
    const size_t nb = (n * 4 + 255) & ~(size_t)255;
    DeviceBlock blk;
    HIP_TRY(hipMalloc((void **)&blk.p, 3 * nb + 256));
    float *d_a = (float *)blk.p, *d_b = (float *)(blk.p + nb), *d_out = (float *)(blk.p + 2 * nb);
    uint32_t *d_err = (uint32_t *)(blk.p + 3 * nb);
    HIP_TRY(hipMemcpy(d_a, a, n * 4, hipMemcpyHostToDevice));
    if (op == 2) HIP_TRY(hipMemcpy(d_b, b, n * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemset(d_err, 0, 256));
    pf_launch_exact_elementwise(op, d_a, d_b, d_out, n, d_err, nullptr);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipMemcpy(error_word, d_err, 4, hipMemcpyDeviceToHost));
    if (*error_word) return PF_HIP_OK;
    HIP_TRY(hipMemcpy(out, d_out, n * 4, hipMemcpyDeviceToHost));
    return PF_HIP_OK;
}

extern "C" int pf_hip_exact_combine_host(const float *down, const uint64_t *pair_to_row, const float *weights,
                                         const float *shared_gate, const float *shared, size_t tokens, size_t top_k,
                                         size_t hidden, float *routed, float *y, uint32_t *error_word) {
    if (!error_word) return PF_HIP_E_ARGUMENT;
    *error_word = 0;
    if (tokens == 0) return PF_HIP_OK;
    if (!down || !pair_to_row || !weights || !shared_gate || !shared || !routed || !y || !top_k || !hidden)
        return PF_HIP_E_ARGUMENT;
    if (tokens * hidden > 0x7fffffffu || tokens * top_k > 0x7fffffffu) return PF_HIP_E_UNSUPPORTED;
    if (need_device()) return PF_HIP_E_NO_DEVICE;
    const size_t pairs = tokens * top_k;
    for (size_t j = 0; j < pairs; j++)
        if (pair_to_row[j] >= pairs) return PF_HIP_E_ARGUMENT;
    auto pad = [](size_t b) { return (b + 255) & ~(size_t)255; };
    const size_t db = pad(pairs * hidden * 4), pb = pad(pairs * 8), wb = pad(pairs * 4), gb = pad(tokens * 4),
                 hb = pad(tokens * hidden * 4);
    DeviceBlock blk;
    HIP_TRY(hipMalloc((void **)&blk.p, db + pb + wb + gb + 3 * hb + 256));
    uint8_t *at = blk.p;
    float *d_down = (float *)at; at += db;
    uint64_t *d_p2r = (uint64_t *)at; at += pb;
    float *d_w = (float *)at; at += wb;
    float *d_sa = (float *)at; at += gb;
    float *d_shared = (float *)at; at += hb;
    float *d_routed = (float *)at; at += hb;
    float *d_y = (float *)at; at += hb;
    uint32_t *d_err = (uint32_t *)at;
    HIP_TRY(hipMemcpy(d_down, down, pairs * hidden * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(d_p2r, pair_to_row, pairs * 8, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(d_w, weights, pairs * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(d_sa, shared_gate, tokens * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(d_shared, shared, tokens * hidden * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemset(d_err, 0, 256));
    pf_launch_exact_combine(d_down, d_p2r, d_w, d_sa, d_shared, d_routed, d_y, (int)tokens, (int)top_k, (int)hidden, d_err,
                            nullptr);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipMemcpy(error_word, d_err, 4, hipMemcpyDeviceToHost));
    // the sums are returned even when flagged: the caller decides which of the two stages failed
    HIP_TRY(hipMemcpy(routed, d_routed, tokens * hidden * 4, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(y, d_y, tokens * hidden * 4, hipMemcpyDeviceToHost));
    return PF_HIP_OK;
}

extern "C" int pf_hip_packed_decode_row_host(uint32_t gguf_type, const void *row, size_t row_bytes, size_t k_storage,
                                             float *out, uint32_t *error_word) {
    if (!error_word) return PF_HIP_E_ARGUMENT;
    *error_word = 0;
    size_t block, size;
    if (!block_geometry(gguf_type, &block, &size)) return PF_HIP_E_UNSUPPORTED;
    if (!row || !out || !k_storage || k_storage > 0x7fffffffu) return PF_HIP_E_ARGUMENT;
    if (need_device()) return PF_HIP_E_NO_DEVICE;
    const uint64_t *grid = pf_device_iq2_grid();
    if (!grid) return PF_HIP_E_MEMORY;
    const size_t wb = (row_bytes + 255) & ~(size_t)255, ob = (k_storage * 4 + 255) & ~(size_t)255;
    DeviceBlock blk;
    HIP_TRY(hipMalloc((void **)&blk.p, wb + ob + 256));
    HIP_TRY(upload_from_host(blk.p, row, row_bytes));
    HIP_TRY(hipMemset(blk.p + wb + ob, 0, 256));
    pf_launch_exact_decode(gguf_type, blk.p, (int)k_storage, (float *)(blk.p + wb), (uint32_t *)(blk.p + wb + ob),
                           grid, nullptr);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipMemcpy(error_word, blk.p + wb + ob, 4, hipMemcpyDeviceToHost));
    if (*error_word) return PF_HIP_OK;
    HIP_TRY(hipMemcpy(out, blk.p + wb, k_storage * 4, hipMemcpyDeviceToHost));
    return PF_HIP_OK;
}

// ---- device memory and timing helpers --------------------------------------------
extern "C" int pf_hip_malloc(void **d_ptr, size_t bytes) {
    if (!d_ptr) return PF_HIP_E_ARGUMENT;
    *d_ptr = nullptr;
    hipError_t e = hipMalloc(d_ptr, bytes ? bytes : 1);
    if (e != hipSuccess) { pf_set_error("hipMalloc", e); return PF_HIP_E_MEMORY; }
    return PF_HIP_OK;
}
extern "C" void pf_hip_free(void *d_ptr) { if (d_ptr) (void)hipFree(d_ptr); }
extern "C" int pf_hip_memcpy_h2d(void *d_dst, const void *src, size_t bytes) {
    HIP_TRY(hipMemcpy(d_dst, src, bytes, hipMemcpyHostToDevice));
    return PF_HIP_OK;
}
extern "C" int pf_hip_memcpy_d2h(void *dst, const void *d_src, size_t bytes) {
    HIP_TRY(hipMemcpy(dst, d_src, bytes, hipMemcpyDeviceToHost));
    return PF_HIP_OK;
}
extern "C" int pf_hip_synchronize(void) {
    HIP_TRY(hipDeviceSynchronize());
    return PF_HIP_OK;
}
