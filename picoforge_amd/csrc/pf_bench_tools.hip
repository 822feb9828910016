// Measuring tools of bench.py: a library of its own (picoforge_amd/libpf_bench.so), not part of the
// shipped one.  It drives libpicoforge_moe.so through its public entry points only
// (include/pf_moe_hip.h) and times with HIP events on the stream the kernels are launched on.
//
// A plan is a sequence of forwards captured once into HIP graphs and replayed as often as wanted: the
// gap between dependent kernels is then the device's, not the host's enqueue rate, and nothing is
// instantiated or destroyed between two timed replays.  A plan of many forwards is one graph of about
// 64 forwards (a whole number of passes over the layers) launched as often as it fits, then one graph
// for the remainder: every kernel node holds its 808-byte argument block, and rocprofv3's kernel trace
// crashed in a graph launch once the nodes of a process added up to more than 1 MiB of them (6144
// nodes did, 960 did not), so a plan keeps to a few hundred nodes whatever its length.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <vector>
#include "pf_bench_tools.h"
#include "pf_moe_debug.h"

static thread_local char g_error[256] = "";
extern "C" const char *pf_bench_last_error(void) { return g_error; }

static int fail(const char *what, hipError_t e) {
    snprintf(g_error, sizeof g_error, "%s: %s", what, hipGetErrorString(e));
    return PF_HIP_E_RUNTIME;
}
#define HIP_TRY(call)                                                     \
    do {                                                                  \
        hipError_t e_ = (call);                                           \
        if (e_ != hipSuccess) return fail(#call, e_);                     \
    } while (0)

struct PfBenchPlan {
    hipStream_t stream = nullptr;
    hipEvent_t t0 = nullptr, t1 = nullptr;
    std::vector<hipGraphExec_t> graphs;   // owned
    std::vector<hipGraphExec_t> launches; // one replay: the graphs in launch order
    void *owned = nullptr;   // device memory the plan's launches use
};

extern "C" void pf_bench_plan_destroy(PfBenchPlan *p) {
    if (!p) return;
    for (hipGraphExec_t g : p->graphs) (void)hipGraphExecDestroy(g);
    if (p->t0) (void)hipEventDestroy(p->t0);
    if (p->t1) (void)hipEventDestroy(p->t1);
    if (p->stream) (void)hipStreamDestroy(p->stream);
    if (p->owned) (void)hipFree(p->owned);
    delete p;
}

static const size_t FORWARDS_PER_GRAPH = 64;

// enqueue(i, stream): forward i of a graph (i counts from 0 in each graph).  period: forwards after which the
// sequence of layers repeats; a graph holds a whole number of periods.
template <typename Enqueue>
static int build_plan(size_t forwards, size_t period, PfBenchPlan **out, Enqueue enqueue) {
    *out = nullptr;
    PfBenchPlan *p = new PfBenchPlan();
    hipError_t e = hipStreamCreate(&p->stream);
    if (e == hipSuccess) e = hipEventCreate(&p->t0);
    if (e == hipSuccess) e = hipEventCreate(&p->t1);
    if (e != hipSuccess) { pf_bench_plan_destroy(p); return fail("plan set-up", e); }
    const size_t unit = period * (FORWARDS_PER_GRAPH / period ? FORWARDS_PER_GRAPH / period : 1);
    const size_t sizes[2] = {forwards >= unit ? unit : 0, forwards % unit}, copies[2] = {forwards / unit, 1};
    int rc = PF_HIP_OK;
    for (int which = 0; which < 2 && rc == PF_HIP_OK; which++) {
        if (!sizes[which]) continue;
        hipGraph_t graph = nullptr;
        hipGraphExec_t exec = nullptr;
        e = hipStreamBeginCapture(p->stream, hipStreamCaptureModeThreadLocal);
        if (e != hipSuccess) { rc = fail("hipStreamBeginCapture", e); break; }
        for (size_t i = 0; i < sizes[which] && rc == PF_HIP_OK; i++) {
            rc = enqueue(i, p->stream);
            if (rc != PF_HIP_OK) snprintf(g_error, sizeof g_error, "forward %zu: shim status %d: %s", i, rc, pf_hip_last_error());
        }
        e = hipStreamEndCapture(p->stream, &graph);
        if (e != hipSuccess && rc == PF_HIP_OK) rc = fail("hipStreamEndCapture", e);
        if (rc == PF_HIP_OK) {
            e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
            if (e != hipSuccess) rc = fail("hipGraphInstantiate", e);
            else {
                p->graphs.push_back(exec);
                for (size_t c = 0; c < copies[which]; c++) p->launches.push_back(exec);
            }
        }
        if (graph) {
            e = hipGraphDestroy(graph);
            if (e != hipSuccess && rc == PF_HIP_OK) rc = fail("hipGraphDestroy", e);
        }
    }
    if (rc != PF_HIP_OK) { pf_bench_plan_destroy(p); return rc; }
    *out = p;
    return PF_HIP_OK;
}

extern "C" int pf_bench_plan_moe(const PfHipMoe *const *moes, PfHipWork *const *works, size_t layers, const float *d_x,
                                 size_t n_inputs, float *d_y, size_t y_blocks, size_t tokens, size_t forwards,
                                 int kernel_limit, size_t hidden, PfBenchPlan **out) {
    if (!out) return PF_HIP_E_ARGUMENT;
    *out = nullptr;
    if (!moes || !works || !layers || !d_x || !d_y || !n_inputs || !y_blocks || !forwards || !hidden) return PF_HIP_E_ARGUMENT;
    for (size_t l = 0; l < layers; l++) {
        if (!moes[l] || !works[l]) return PF_HIP_E_ARGUMENT;
        pf_hip_work_limit_kernels(works[l], kernel_limit);
    }
    const size_t block = tokens * hidden;
    const int rc = build_plan(forwards, layers, out, [&](size_t i, hipStream_t s) {
        return pf_hip_moe_forward_device(moes[i % layers], works[i % layers], d_x + (i % n_inputs) * block, hidden,
                                         d_y + (i % y_blocks) * block, hidden, tokens, s);
    });
    for (size_t l = 0; l < layers; l++) pf_hip_work_limit_kernels(works[l], 0);
    return rc;
}

extern "C" int pf_bench_plan_hc(const PfHipMoe *moe, PfHipWork *work, const float *d_normed, const float *d_logits,
                                size_t n_inputs, float *d_residual, const float *d_inject, size_t streams, size_t tokens,
                                size_t forwards, int fused, size_t hidden, PfBenchPlan **out) {
    if (!out) return PF_HIP_E_ARGUMENT;
    *out = nullptr;
    if (!moe || !work || !d_normed || !d_logits || !d_residual || !d_inject || !n_inputs || !streams || !forwards || !hidden)
        return PF_HIP_E_ARGUMENT;
    const size_t H = hidden, cube = tokens * streams * H;
    // the unfused chain needs rows for the mixed input and the block's output between its three enqueues
    float *rows = nullptr;
    if (!fused) HIP_TRY(hipMalloc((void **)&rows, 2 * tokens * H * sizeof(float)));
    const int rc = build_plan(forwards, 1, out, [&](size_t i, hipStream_t s) {
        const float *n = d_normed + (i % n_inputs) * cube, *g = d_logits + (i % n_inputs) * cube;
        if (fused)
            return pf_hip_moe_forward_hc_device(moe, work, n, streams * H, H, g, streams * H, H, d_residual, streams * H, H,
                                                d_inject, streams, tokens, s);
        uint32_t *err = const_cast<uint32_t *>(pf_hip_work_error_word(work));
        int r = pf_hip_hc_read_device(n, streams * H, H, g, streams * H, H, rows, H, tokens, streams, H, err, s);
        if (r == PF_HIP_OK) r = pf_hip_moe_forward_device(moe, work, rows, H, rows + tokens * H, H, tokens, s);
        if (r == PF_HIP_OK)
            r = pf_hip_hc_add_device(d_residual, streams * H, H, rows + tokens * H, H, d_inject, streams, tokens, streams, H, err, s);
        return r;
    });
    if (rc == PF_HIP_OK) (*out)->owned = rows;
    else if (rows) (void)hipFree(rows);
    return rc;
}

extern "C" int pf_bench_plan_run(PfBenchPlan *p, size_t repeats, float *ms_each) {
    if (!p || !repeats || !ms_each) return PF_HIP_E_ARGUMENT;
    for (size_t r = 0; r < repeats; r++) {
        HIP_TRY(hipEventRecord(p->t0, p->stream));
        for (hipGraphExec_t g : p->launches) HIP_TRY(hipGraphLaunch(g, p->stream));
        HIP_TRY(hipEventRecord(p->t1, p->stream));
        HIP_TRY(hipStreamSynchronize(p->stream));
        HIP_TRY(hipEventElapsedTime(&ms_each[r], p->t0, p->t1));
    }
    return PF_HIP_OK;
}

// One of the two hyper-connection kernels alone, `iters` launches back to back on a stream of its own,
// bracketed by two events on that stream.  which 0: the read (dense inputs, output into d_rows);
// which 1: the add of d_rows into d_cube (dense), weights d_inject.
extern "C" int pf_bench_hc_time_step(int which, float *d_cube, const float *d_logits, float *d_rows, const float *d_inject,
                                     size_t tokens, size_t streams, size_t hidden, size_t iters, uint32_t *d_error_word,
                                     float *elapsed_ms) {
    if (!d_cube || !d_rows || !elapsed_ms || !d_error_word || !tokens || !streams || !hidden || (which == 0 ? !d_logits : !d_inject))
        return PF_HIP_E_ARGUMENT;
    hipStream_t s = nullptr;
    hipEvent_t t0 = nullptr, t1 = nullptr;
    HIP_TRY(hipStreamCreate(&s));
    hipError_t e = hipEventCreate(&t0);
    if (e == hipSuccess) e = hipEventCreate(&t1);
    if (e == hipSuccess) e = hipEventRecord(t0, s);
    int rc = PF_HIP_OK;
    for (size_t i = 0; i < iters && e == hipSuccess && rc == PF_HIP_OK; i++) {
        if (which == 0)
            rc = pf_hip_hc_read_device(d_cube, streams * hidden, hidden, d_logits, streams * hidden, hidden, d_rows, hidden, tokens,
                                       streams, hidden, d_error_word, s);
        else
            rc = pf_hip_hc_add_device(d_cube, streams * hidden, hidden, d_rows, hidden, d_inject, streams, tokens, streams, hidden,
                                      d_error_word, s);
    }
    if (e == hipSuccess) e = hipEventRecord(t1, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e == hipSuccess) e = hipEventElapsedTime(elapsed_ms, t0, t1);
    if (t0) (void)hipEventDestroy(t0);
    if (t1) (void)hipEventDestroy(t1);
    (void)hipStreamDestroy(s);
    if (e != hipSuccess) return fail("timed hyper-connection kernel", e);
    return rc;
}

// A plain copy of a known size: the reference point for hardware byte counters, which a profiler
// reads in units that are easiest to pin against a kernel whose traffic is known.
__global__ void pf_k_copy_probe(const uint4 *src, uint4 *dst, size_t count) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x)
        dst[i] = src[i];
}

extern "C" int pf_bench_copy_probe(size_t bytes, size_t launches) {
    bytes &= ~(size_t)15;
    if (!bytes || !launches) return PF_HIP_E_ARGUMENT;
    uint4 *src = nullptr, *dst = nullptr;
    hipError_t e = hipMalloc((void **)&src, bytes);
    if (e == hipSuccess) e = hipMalloc((void **)&dst, bytes);
    if (e == hipSuccess) e = hipMemset(src, 1, bytes);
    for (size_t i = 0; i < launches && e == hipSuccess; i++) {
        hipLaunchKernelGGL(pf_k_copy_probe, dim3(2048), dim3(256), 0, nullptr, src, dst, bytes / 16);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (src) (void)hipFree(src);
    if (dst) (void)hipFree(dst);
    return e == hipSuccess ? PF_HIP_OK : fail("copy probe", e);
}
