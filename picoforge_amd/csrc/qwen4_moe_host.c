/* C11 host side of the MoE block (include/qwen4_moe.h): handles, lifecycle and
 * the reference's preflight validation in the reference's order
 * (src/qwen4_moe.c), so that callers and tests see the same status codes.  All
 * arithmetic is done by the HIP kernels behind include/pf_moe_hip.h; there is no
 * CPU fallback: without a device every compute entry point fails. */
#include "../../include/qwen4_moe.h"
#include "../../include/qwen4_hc.h"
#include "../../include/qwen4_expert_pool.h"
#include "../../include/pf_moe_hip.h"
#include "pf_hc_host.h"
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

Qwen4Status pf_packed_admit(const QW4PackedCpuView *w, size_t expert);              /* qwen4_packed_host.c */
Qwen4Status pf_layout_admit(const QW4PackedLayout *l);
Qwen4Status pf_device_status(int rc, Qwen4Error *err, const char *subject);

typedef struct { uintptr_t lo, hi; } Range;

struct Qwen4Moe {
    Qwen4MoeConfig cfg;
    QW4PackedCpuView w[8];
    size_t refs;
    bool alive;
    PfHipMoe *device;
    PfHipMoeDesc desc;
    bool host_spans;   /* the caller still holds the weight bytes at w[].span (the reference's contract) */
    bool streamed;     /* the routed tensors are read from an expert pool, forward by forward */
    FILE *route_log;   /* PF_ROUTE_LOG: this layer's routed ids, one record per forward */
    uint64_t route_pos;
};

struct Qwen4MoeWork {
    Qwen4Moe *owner;
    size_t cap, bytes;
    PfHipWork *device;
    bool busy, failed;
    QW4MoeObserver observer;
    void *observer_ctx;
};

static Qwen4Status moe_status(Qwen4Error *err, Qwen4Status code, const char *detail) {
    if (err) {
        memset(err, 0, sizeof *err);
        err->code = code;
        if (code != QW4_OK) {
            snprintf(err->subject, sizeof err->subject, "qwen4_moe");
            snprintf(err->detail, sizeof err->detail, "%s", detail);
        }
    }
    return code;
}
#define TRY(expr) do { Qwen4Status st_ = (expr); if (st_ != QW4_OK) return st_; } while (0)

static Qwen4Status admit_config(const Qwen4MoeConfig *c, Qwen4Error *err) {
    if (!c) return moe_status(err, QW4_INVALID_ARGUMENT, "null config");
    if (!c->hidden_size || !c->experts || !c->top_k || c->top_k > c->experts || !c->intermediate ||
        !c->shared_intermediate || c->down_physical < c->intermediate)
        return moe_status(err, QW4_RANGE, "invalid MoE dimensions");
    return QW4_OK;
}

/* ---- routing trace (the per-layer part of QW4_ROUTE_LOG, src/qwen4_forward_gpu.m:62-65,369-376,894-900) ----
 * Off unless PF_ROUTE_LOG is set.  The n-th layer this process creates (n from 0) appends to the new
 * file "<PF_ROUTE_LOG>.<n>" one record per forward in the reference's record format with one layer:
 * uint32 pos, count, layers = 1, top_k, then uint32 ids [count][top_k]; pos is the number of tokens
 * the layer has been given before the call.  Never read by the forward itself. */
static unsigned route_log_layers;

static Qwen4Status route_log_open(Qwen4Moe *m, Qwen4Error *err) {
    const char *prefix = getenv("PF_ROUTE_LOG");
    if (!prefix || !*prefix) return QW4_OK;
    char path[4096];
    if (snprintf(path, sizeof path, "%s.%u", prefix, route_log_layers) >= (int)sizeof path)
        return moe_status(err, QW4_INVALID_ARGUMENT, "PF_ROUTE_LOG path too long");
    m->route_log = fopen(path, "wbx");
    if (!m->route_log) return moe_status(err, QW4_IO, "route log (PF_ROUTE_LOG.<layer> must name a new file)");
    route_log_layers++;
    return QW4_OK;
}

static void route_log_append(Qwen4Moe *m, const uint32_t *ids, size_t pitch_words, size_t tokens) {
    const uint32_t head[4] = {(uint32_t)m->route_pos, (uint32_t)tokens, 1u, m->cfg.top_k};
    fwrite(head, 4, 4, m->route_log);
    for (size_t t = 0; t < tokens; t++) fwrite(ids + t * pitch_words, 4, m->cfg.top_k, m->route_log);
    fflush(m->route_log);
    m->route_pos += tokens;
}

/* ---- create / destroy ------------------------------------------------------ */
static Qwen4Status create_layer(const Qwen4MoeConfig *c, const Qwen4MoeWeights *weights, bool streamed, Qwen4Moe **out,
                                Qwen4Error *err) {
    if (out) *out = NULL;
    if (!out || !weights) return moe_status(err, QW4_INVALID_ARGUMENT, "null create argument");
    TRY(admit_config(c, err));
    const QW4PackedCpuView w[8] = {weights->router, weights->gate, weights->up, weights->down,
                                   weights->shared_gate, weights->shared_up, weights->shared_down,
                                   weights->shared_router};
    const size_t h = c->hidden_size, i = c->intermediate, s = c->shared_intermediate;
    const size_t k_in[8] = {h, h, h, i, h, h, s, h}, n_out[8] = {c->experts, i, i, h, s, s, h, 1};
    for (size_t a = 0; a < 8; a++) {
        const QW4PackedLayout *l = &w[a].layout;
        const size_t experts = (a >= 1 && a <= 3) ? c->experts : 1;
        if (l->k_logical != k_in[a] || l->n_out != n_out[a] || l->n_experts != experts ||
            l->k_storage != (a == 3 ? c->down_physical : k_in[a]))
            return moe_status(err, QW4_SHAPE, "MoE weight shape mismatch");
        if ((a == 0 || a == 7) && l->gguf_type != 0) return moe_status(err, QW4_FORMAT, "router must be F32");
        const bool on_disk = streamed && a >= 1 && a <= 3;
        if (on_disk && w[a].span.data) return moe_status(err, QW4_INVALID_ARGUMENT, "a streamed layer takes no routed bytes");
        Qwen4Status st = on_disk ? pf_layout_admit(l) : pf_packed_admit(&w[a], 0);
        if (st) {
            moe_status(err, st, "invalid weight view");
            if (err) snprintf(err->subject, sizeof err->subject, "packed weights");
            return st;
        }
    }
    Qwen4Moe *m = calloc(1, sizeof *m);
    if (!m) return moe_status(err, QW4_OOM, "MoE allocation");
    m->cfg = *c;
    memcpy(m->w, w, sizeof w);
    m->desc = (PfHipMoeDesc){.hidden = c->hidden_size, .experts = c->experts, .top_k = c->top_k,
                             .inter = c->intermediate, .shared_inter = c->shared_intermediate,
                             .down_physical = c->down_physical, .norm_topk = c->norm_topk_prob ? 1u : 0u};
    const void *bytes[8];
    size_t sizes[8];
    for (size_t a = 0; a < 8; a++) {
        m->desc.type[a] = w[a].layout.gguf_type;
        bytes[a] = w[a].span.data;
        sizes[a] = w[a].layout.tensor_bytes;
    }
    int rc = pf_hip_moe_create(&m->desc, bytes, sizes, &m->device);
    if (rc) { free(m); return pf_device_status(rc, err, "qwen4_moe"); }
    m->refs = 1;
    m->alive = true;
    m->host_spans = true;
    m->streamed = streamed;
    Qwen4Status st = route_log_open(m, err);
    if (st) { pf_hip_moe_destroy(m->device); free(m); return st; }
    *out = m;
    return moe_status(err, QW4_OK, "");
}

Qwen4Status qwen4_moe_create(const Qwen4MoeConfig *c, const Qwen4MoeWeights *weights, Qwen4Moe **out,
                             Qwen4Error *err) {
    return create_layer(c, weights, false, out, err);
}

/* A layer for models larger than device memory: router, shared expert and shared router resident, the
 * routed gate, up and down tensors left in the model file (their views carry layouts and no bytes). */
Qwen4Status pf_moe_create_streamed(const Qwen4MoeConfig *c, const Qwen4MoeWeights *weights, Qwen4Moe **out,
                                   Qwen4Error *err) {
    return create_layer(c, weights, true, out, err);
}

static void moe_unref(Qwen4Moe *m) {
    if (m && --m->refs == 0) {
        if (m->route_log) fclose(m->route_log);
        pf_hip_moe_destroy(m->device);
        free(m);
    }
}
void qwen4_moe_destroy(Qwen4Moe *m) {
    if (m && m->alive) { m->alive = false; moe_unref(m); }
}

/* ---- workspaces ------------------------------------------------------------ */
static Qwen4Status plan_work(const Qwen4Moe *m, size_t cap, size_t *bytes, Qwen4Error *err) {
    if (!m || !m->alive) return moe_status(err, QW4_BAD_STATE, "inactive MoE");
    const size_t k = m->cfg.top_k, widest = (size_t)m->cfg.hidden_size + m->cfg.experts + k * m->cfg.intermediate;
    if (cap > SIZE_MAX / 64 / (widest ? widest : 1)) return moe_status(err, QW4_OVERFLOW, "scratch size overflow");
    *bytes = sizeof(Qwen4MoeWork) + pf_hip_work_bytes(&m->desc, cap);
    return QW4_OK;
}

Qwen4Status qwen4_moe_work_size(const Qwen4Moe *m, size_t cap, size_t *bytes, Qwen4Error *err) {
    if (!bytes) return moe_status(err, QW4_INVALID_ARGUMENT, "null size output");
    *bytes = 0;
    size_t need;
    TRY(plan_work(m, cap, &need, err));
    *bytes = need;
    return moe_status(err, QW4_OK, "");
}

Qwen4Status qwen4_moe_work_create(const Qwen4Moe *m, size_t cap, size_t budget, Qwen4MoeWork **out, Qwen4Error *err) {
    if (out) *out = NULL;
    if (!out) return moe_status(err, QW4_INVALID_ARGUMENT, "null workspace output");
    size_t need;
    TRY(plan_work(m, cap, &need, err));
    if (budget < need) return moe_status(err, QW4_CAPACITY, "workspace budget too small");
    Qwen4MoeWork *w = calloc(1, sizeof *w);
    if (!w) return moe_status(err, QW4_OOM, "workspace metadata");
    int rc = pf_hip_work_create(m->device, cap, &w->device);
    if (rc) { free(w); return pf_device_status(rc, err, "qwen4_moe"); }
    w->owner = (Qwen4Moe *)m;
    w->owner->refs++;
    w->cap = cap;
    w->bytes = need;
    *out = w;
    return moe_status(err, QW4_OK, "");
}

Qwen4Status qwen4_moe_work_reset(Qwen4MoeWork *w, Qwen4Error *err) {
    if (!w) return moe_status(err, QW4_INVALID_ARGUMENT, "null workspace");
    if (w->busy) return moe_status(err, QW4_BUSY, "workspace executing");
    if (!w->owner->alive) return moe_status(err, QW4_BAD_STATE, "destroyed owner");
    w->failed = false;
    return moe_status(err, QW4_OK, "");
}

void qwen4_moe_work_destroy(Qwen4MoeWork *w) {
    if (w && !w->busy) { pf_hip_work_destroy(w->device); moe_unref(w->owner); free(w); }
}

/* The weights live in device memory from create on.  A caller that frees or unmaps its host bytes
 * before destroy (which the reference's borrowing contract, src/qwen4_moe.h:12, does not allow) says
 * so here: forward then no longer compares its views with the addresses the bytes once had, which
 * another allocation may own by then. */
void pf_moe_forget_host_weights(Qwen4Moe *m) {
    if (m) m->host_spans = false;
}

PfHipMoe *pf_moe_device_layer(const Qwen4Moe *m) { return m ? m->device : NULL; }
PfHipWork *pf_moe_device_work(Qwen4MoeWork *w) { return w ? w->device : NULL; }

void qw4_moe_observe(Qwen4MoeWork *w, QW4MoeObserver fn, void *ctx) {
    if (w && !w->busy) { w->observer = fn; w->observer_ctx = ctx; }
}

/* ---- view admission (src/qwen4_moe.c:134-186) --------------------------------- */
static Qwen4Status range_of(const void *data, size_t cap, size_t bytes, size_t alignment, Range *r, Qwen4Error *err) {
    r->lo = r->hi = 0;
    if (!bytes) return QW4_OK;
    if (cap < bytes) return moe_status(err, QW4_CAPACITY, "view capacity too small");
    if (!data) return moe_status(err, QW4_INVALID_ARGUMENT, "null nonempty view");
    uintptr_t lo = (uintptr_t)data;
    if (lo % alignment) return moe_status(err, QW4_STRIDE, "unaligned view");
    if (bytes > UINTPTR_MAX - lo) return moe_status(err, QW4_OVERFLOW, "address extent overflow");
    r->lo = lo;
    r->hi = lo + bytes;
    return QW4_OK;
}

static Qwen4Status range_rows(const void *data, size_t cap, size_t rows, size_t cols, size_t pitch, Range *r,
                              Qwen4Error *err) {
    r->lo = r->hi = 0;
    if (cols > SIZE_MAX / 4) return moe_status(err, QW4_OVERFLOW, "row bytes overflow");
    const size_t row_bytes = cols * 4;
    if (pitch % 4 || pitch < row_bytes)
        return moe_status(err, QW4_STRIDE, "row stride must cover contiguous features");
    if (!rows) return QW4_OK;
    if (rows - 1 > (SIZE_MAX - row_bytes) / pitch) return moe_status(err, QW4_OVERFLOW, "view extent overflow");
    return range_of(data, cap, (rows - 1) * pitch + row_bytes, 4, r, err);
}

static Qwen4Status range_f32(const float *data, size_t cap, size_t rank, const size_t dim[4], const size_t stride[4],
                             size_t rows, size_t cols, Range *r, Qwen4Error *err) {
    if (rank != 2 || dim[0] != rows || dim[1] != cols)
        return moe_status(err, QW4_SHAPE, "expected rank-2 token-major view");
    if (stride[1] != sizeof(float)) return moe_status(err, QW4_STRIDE, "features must be contiguous");
    return range_rows(data, cap, rows, cols, stride[0], r, err);
}
#define RANGE_F32(v, rows, cols, r) \
    range_f32((v).data, (v).capacity_bytes, (v).rank, (v).dim, (v).stride_bytes, rows, cols, r, err)

static Qwen4Status all_disjoint(const Range *r, size_t n, Qwen4Error *err) {
    for (size_t i = 0; i < n; i++)
        for (size_t j = 0; j < i; j++)
            if (r[i].lo < r[j].hi && r[j].lo < r[i].hi)
                return moe_status(err, QW4_INVALID_ARGUMENT, "overlapping views");
    return QW4_OK;
}

/* ---- routing on caller-provided logits ------------------------------------------ */
Qwen4Status qwen4_moe_route(const Qwen4MoeConfig *c, Qwen4F32 logits, Qwen4MoeRoutes routes,
                            Qwen4F32Mut probabilities, Qwen4Error *err) {
    TRY(admit_config(c, err));
    const size_t T = logits.dim[0], E = c->experts, K = c->top_k;
    Range r[4];
    TRY(RANGE_F32(logits, T, E, &r[0]));
    TRY(RANGE_F32(probabilities, T, E, &r[1]));
    TRY(RANGE_F32(routes.weights, T, K, &r[2]));
    if (routes.ids.rows != T || routes.ids.cols != K) return moe_status(err, QW4_SHAPE, "route ID shape mismatch");
    TRY(range_rows(routes.ids.data, routes.ids.capacity_bytes, T, K, routes.ids.row_stride_bytes, &r[3], err));
    TRY(all_disjoint(r, 4, err));
    if (!T) return moe_status(err, QW4_OK, "");
    float *z = malloc(T * E * 4), *p = malloc(T * E * 4), *w = malloc(T * K * 4);
    uint32_t *ids = malloc(T * K * 4);
    Qwen4Status st = QW4_OK;
    if (!z || !p || !w || !ids) st = moe_status(err, QW4_OOM, "route staging");
    if (!st) {
        for (size_t t = 0; t < T; t++) memcpy(z + t * E, logits.data + t * (logits.stride_bytes[0] / 4), E * 4);
        uint32_t word = 0;
        uint64_t bad_row = 0;
        int rc = pf_hip_route_host(z, T, E, K, c->norm_topk_prob, p, ids, w, &word, &bad_row);
        if (rc) st = pf_device_status(rc, err, "qwen4_moe");
        else if (word & PF_HIP_ERR_NONFINITE) {
            st = moe_status(err, QW4_NONFINITE, "nonfinite router logit");
            if (err) err->row = bad_row;
        } else if (word) st = moe_status(err, QW4_GPU_ERROR, "device error word");
    }
    if (!st) {
        for (size_t t = 0; t < T; t++) {
            memcpy(probabilities.data + t * (probabilities.stride_bytes[0] / 4), p + t * E, E * 4);
            memcpy(routes.weights.data + t * (routes.weights.stride_bytes[0] / 4), w + t * K, K * 4);
            memcpy(routes.ids.data + t * (routes.ids.row_stride_bytes / 4), ids + t * K, K * 4);
        }
        moe_status(err, QW4_OK, "");
    }
    free(z); free(p); free(w); free(ids);
    return st;
}

/* ---- grouping ---------------------------------------------------------------------- */
Qwen4Status qw4_moe_group_pairs(const Qwen4MoeConfig *c, Qwen4U32Mut ids, QW4MoeGrouping g, Qwen4Error *err) {
    TRY(admit_config(c, err));
    if (ids.cols != c->top_k) return moe_status(err, QW4_SHAPE, "group ID shape mismatch");
    const size_t E = c->experts, K = c->top_k;
    if (ids.rows > SIZE_MAX / K || E == SIZE_MAX) return moe_status(err, QW4_OVERFLOW, "group count overflow");
    const size_t pairs = ids.rows * K;
    Range r[5];
    TRY(range_rows(ids.data, ids.capacity_bytes, ids.rows, ids.cols, ids.row_stride_bytes, &r[0], err));
    const void *ptr[4] = {g.offsets, g.cursors, g.pair_to_row, g.row_to_pair};
    const size_t count[4] = {E + 1, E, pairs, pairs};
    const size_t cap[4] = {g.offsets_capacity_bytes, g.cursors_capacity_bytes, g.pair_to_row_capacity_bytes,
                           g.row_to_pair_capacity_bytes};
    for (size_t a = 0; a < 4; a++) {
        if (count[a] > SIZE_MAX / sizeof(size_t)) return moe_status(err, QW4_OVERFLOW, "group array bytes overflow");
        TRY(range_of(ptr[a], cap[a], count[a] * sizeof(size_t), _Alignof(size_t), &r[a + 1], err));
    }
    TRY(all_disjoint(r, 5, err));
    _Static_assert(sizeof(size_t) == sizeof(uint64_t), "the shim exchanges 64-bit indices");
    uint32_t *dense = NULL;
    if (pairs) {
        dense = malloc(pairs * 4);
        if (!dense) return moe_status(err, QW4_OOM, "group staging");
        for (size_t t = 0; t < ids.rows; t++) memcpy(dense + t * K, ids.data + t * (ids.row_stride_bytes / 4), K * 4);
    }
    uint64_t *out = malloc((E + 1 + 2 * pairs) * sizeof(uint64_t));
    if (!out) { free(dense); return moe_status(err, QW4_OOM, "group staging"); }
    uint32_t word = 0;
    int duplicate = 0;
    int rc = pf_hip_group_pairs_host(dense, ids.rows, E, K, out, out + E + 1, out + E + 1 + pairs, &word, &duplicate);
    Qwen4Status st;
    if (rc) st = pf_device_status(rc, err, "qwen4_moe");
    else if (word & PF_HIP_ERR_BOUNDS) st = moe_status(err, QW4_RANGE, "expert ID out of range");
    else if (duplicate) st = moe_status(err, QW4_INVALID_ARGUMENT, "duplicate expert ID");
    else {
        memcpy(g.offsets, out, (E + 1) * sizeof(size_t));
        for (size_t e = 0; e < E; e++) g.cursors[e] = (size_t)out[e + 1];   /* cursors end at offsets[e+1] */
        if (pairs) {
            memcpy(g.pair_to_row, out + E + 1, pairs * sizeof(size_t));
            memcpy(g.row_to_pair, out + E + 1 + pairs, pairs * sizeof(size_t));
        }
        st = moe_status(err, QW4_OK, "");
    }
    free(out);
    free(dense);
    return st;
}

/* ---- the observed forward (src/qwen4_moe.c:305-382) -------------------------------------------
 * With an observer set the block runs as the reference's sequence of operators, one device call each
 * in the reference's evaluation order, in microbatches of at most 32 tokens, and every stage's input
 * and output rows are handed to the observer from host staging memory.  This is the slow, bit-identical
 * mode: it reads each expert's bytes from the caller's host views on every call, so it needs them. */
typedef struct {
    float *z, *p, *scores, *gather, *down, *gate, *up, *act, *shared, *sg, *sa, *routed, *yd;
    uint32_t *ids;
    size_t *offsets, *cursors, *p2r, *r2p;
} Stage;

static Qwen4F32Mut rows_of(float *data, size_t rows, size_t cols) {
    return (Qwen4F32Mut){.data = data, .capacity_bytes = rows * cols * 4, .rank = 2, .dim = {rows, cols},
                         .stride_bytes = {cols * 4, 4}};
}
static Qwen4F32 ro(Qwen4F32Mut v) {
    Qwen4F32 r = {.data = v.data, .capacity_bytes = v.capacity_bytes, .rank = v.rank};
    memcpy(r.dim, v.dim, sizeof r.dim);
    memcpy(r.stride_bytes, v.stride_bytes, sizeof r.stride_bytes);
    return r;
}
static void trace(Qwen4MoeWork *w, size_t stage, size_t expert, size_t token, Qwen4F32 in, Qwen4F32Mut out) {
    w->observer(w->observer_ctx, stage, expert, token, in, ro(out));
}
static Qwen4Status linear(Qwen4MoeWork *w, size_t stage, size_t expert, size_t token, Qwen4F32 x, Qwen4F32Mut y,
                          Qwen4Error *err) {
    TRY(qw4_packed_matmul(&w->owner->w[stage], expert, x, y, err));
    trace(w, stage, expert, token, x, y);
    return QW4_OK;
}
static Qwen4Status elementwise(int op, const float *a, const float *b, size_t n, float *out, const char *what,
                               Qwen4Error *err) {
    uint32_t word = 0;
    int rc = pf_hip_exact_elementwise_host(op, a, b, n, out, &word);
    if (rc) return pf_device_status(rc, err, "qwen4_moe");
    if (word & PF_HIP_ERR_NONFINITE) return moe_status(err, QW4_NONFINITE, what);
    return word ? moe_status(err, QW4_GPU_ERROR, "device error word") : QW4_OK;
}

static Qwen4Status observed_expert(Qwen4MoeWork *w, Stage *b, size_t expert, size_t token, Qwen4F32 x, Qwen4F32Mut y,
                                   bool shared, Qwen4Error *err) {
    const Qwen4MoeConfig *c = &w->owner->cfg;
    const size_t n = x.dim[0], i = shared ? c->shared_intermediate : c->intermediate;
    const size_t who = shared ? SIZE_MAX : expert;
    Qwen4F32Mut g = rows_of(b->gate, n, i), u = rows_of(b->up, n, i), a = rows_of(b->act, n, i);
    TRY(linear(w, shared ? 4 : 1, expert, token, x, g, err));
    TRY(linear(w, shared ? 5 : 2, expert, token, x, u, err));
    TRY(elementwise(0, g.data, NULL, n * i, a.data, "activation overflow", err));
    trace(w, 8, who, token, ro(g), a);
    TRY(elementwise(2, a.data, u.data, n * i, a.data, "gate/up overflow", err));
    trace(w, 9, who, token, ro(u), a);
    return linear(w, shared ? 6 : 3, expert, token, ro(a), y, err);
}

static Qwen4Status observed_batch(Qwen4MoeWork *w, Stage *b, Qwen4F32 x, Qwen4F32Mut y, size_t token, Qwen4Error *err) {
    const Qwen4MoeConfig *c = &w->owner->cfg;
    const size_t t = x.dim[0], e = c->experts, k = c->top_k, h = c->hidden_size, pairs = t * k;
    Qwen4F32Mut z = rows_of(b->z, t, e), p = rows_of(b->p, t, e);
    Qwen4MoeRoutes routes = {{b->ids, pairs * 4, t, k, k * 4}, rows_of(b->scores, t, k)};
    TRY(linear(w, 0, 0, token, x, z, err));
    TRY(qwen4_moe_route(c, ro(z), routes, p, err));
    QW4MoeGrouping g = {b->offsets, (e + 1) * sizeof(size_t), b->cursors, e * sizeof(size_t), b->p2r, b->r2p,
                        pairs * sizeof(size_t), pairs * sizeof(size_t)};
    TRY(qw4_moe_group_pairs(c, routes.ids, g, err));
    for (size_t row = 0; row < pairs; row++)
        memcpy(b->gather + row * h, x.data + (g.row_to_pair[row] / k) * (x.stride_bytes[0] / 4), h * 4);
    for (size_t expert = 0; expert < e; expert++) {
        const size_t first = g.offsets[expert], n = g.offsets[expert + 1] - first;
        if (!n) continue;
        TRY(observed_expert(w, b, expert, token, ro(rows_of(b->gather + first * h, n, h)), rows_of(b->down + first * h, n, h),
                            false, err));
    }
    Qwen4F32Mut shared = rows_of(b->shared, t, h), sg = rows_of(b->sg, t, 1), sa = rows_of(b->sa, t, 1);
    TRY(observed_expert(w, b, 0, token, x, shared, true, err));
    TRY(linear(w, 7, 0, token, x, sg, err));
    TRY(elementwise(1, sg.data, NULL, t, sa.data, "activation overflow", err));
    trace(w, 10, SIZE_MAX, token, ro(sg), sa);
    uint32_t word = 0;
    _Static_assert(sizeof(size_t) == sizeof(uint64_t), "the shim exchanges 64-bit indices");
    int rc = pf_hip_exact_combine_host(b->down, (const uint64_t *)g.pair_to_row, b->scores, b->sa, b->shared, t, k, h,
                                       b->routed, b->yd, &word);
    if (rc) return pf_device_status(rc, err, "qwen4_moe");
    if (word & ~PF_HIP_ERR_NONFINITE) return moe_status(err, QW4_GPU_ERROR, "device error word");
    const size_t ys = y.stride_bytes[0] / 4;
    if (word)   /* a nonfinite routed sum fails before stage 11, anything later after it */
        for (size_t j = 0; j < t * h; j++)
            if (!isfinite(b->routed[j])) return moe_status(err, QW4_NONFINITE, "routed reduction overflow");
    for (size_t row = 0; row < t; row++) memcpy(y.data + row * ys, b->routed + row * h, h * 4);
    trace(w, 11, SIZE_MAX, token, x, y);
    if (word) return moe_status(err, QW4_NONFINITE, "shared sum overflow");
    for (size_t row = 0; row < t; row++) memcpy(y.data + row * ys, b->yd + row * h, h * 4);
    trace(w, 12, SIZE_MAX, token, x, y);
    return QW4_OK;
}

static Qwen4Status observed_forward(Qwen4MoeWork *w, Qwen4F32 x, Qwen4F32Mut y, Qwen4MoeRoutes *routes, Qwen4Error *err) {
    const Qwen4MoeConfig *c = &w->owner->cfg;
    if (!w->owner->host_spans) return moe_status(err, QW4_BAD_STATE, "the observer needs the host weight bytes");
    const size_t T = x.dim[0], micro = w->cap < 32 ? w->cap : 32, e = c->experts, k = c->top_k, h = c->hidden_size;
    const size_t i = c->intermediate > c->shared_intermediate ? c->intermediate : c->shared_intermediate;
    const size_t pairs = micro * k;
    const size_t floats[13] = {micro * e, micro * e, pairs, pairs * h, pairs * h, micro * i, micro * i, micro * i,
                               micro * h, micro, micro, micro * h, micro * h};
    size_t total = 0;
    for (size_t j = 0; j < 13; j++) total += floats[j];
    float *arena = malloc((total ? total : 1) * 4);
    uint32_t *ids = malloc((pairs ? pairs : 1) * 4);
    size_t *index = malloc((2 * e + 1 + 2 * pairs) * sizeof(size_t));
    Qwen4Status st = QW4_OK;
    if (!arena || !ids || !index) st = moe_status(err, QW4_OOM, "observer staging");
    if (!st) {
        float *at = arena;
        Stage b = {.ids = ids, .offsets = index, .cursors = index + e + 1, .p2r = index + 2 * e + 1,
                   .r2p = index + 2 * e + 1 + pairs};
        float **fields[13] = {&b.z, &b.p, &b.scores, &b.gather, &b.down, &b.gate, &b.up, &b.act, &b.shared, &b.sg, &b.sa,
                              &b.routed, &b.yd};
        for (size_t j = 0; j < 13; j++) { *fields[j] = at; at += floats[j]; }
        for (size_t start = 0; start < T && !st;) {
            const size_t n = T - start < micro ? T - start : micro;
            Qwen4F32 bx = x;
            Qwen4F32Mut by = y;
            bx.data += start * (x.stride_bytes[0] / 4); bx.capacity_bytes -= start * x.stride_bytes[0]; bx.dim[0] = n;
            by.data += start * (y.stride_bytes[0] / 4); by.capacity_bytes -= start * y.stride_bytes[0]; by.dim[0] = n;
            st = observed_batch(w, &b, bx, by, start, err);
            if (!st && routes)
                for (size_t row = 0; row < n; row++) {
                    memcpy(routes->ids.data + (start + row) * (routes->ids.row_stride_bytes / 4), b.ids + row * k, k * 4);
                    memcpy(routes->weights.data + (start + row) * (routes->weights.stride_bytes[0] / 4), b.scores + row * k,
                           k * 4);
                }
            start += n;
        }
    }
    free(arena); free(ids); free(index);
    return st ? st : moe_status(err, QW4_OK, "");
}

/* ---- forward (src/qwen4_moe.c:384-431) -------------------------------------------------- */
/* The two device calls of a streamed layer with the pool between them (the reference's remap hook,
 * src/qwen4_moe_internal.h:49-54, and its caller's acquire/release, src/qwen4_forward_gpu.m). */
static Qwen4Status streamed_forward(const Qwen4Moe *m, Qwen4MoeWork *w, QW4ExpertPool *pool, uint32_t layer, Qwen4F32 x,
                                    Qwen4F32Mut y, Qwen4MoeRoutes *routes, Qwen4Error *err) {
    const size_t T = x.dim[0], K = m->cfg.top_k, pairs = T * K;
    const void *regions[3];
    size_t expert_bytes[3], scale_offsets[3];
    const size_t pool_slots = pf_pool_slots(pool);
    uint32_t tiled_mask = 0;   /* regions whose slots the pool stored in the Q4_K tile order */
    for (int j = 0; j < 3; j++) {
        const QW4PackedLayout *l = &m->w[1 + j].layout;
        const uint32_t format = pf_pool_format(pool, j);
        if (format != UINT32_MAX && pf_hip_pool_slot_tiled(l->gguf_type, l->n_out)) tiled_mask |= 1u << j;
        size_t region_bytes = 0, want_bytes = 0, file_bytes = 0;
        regions[j] = qw4_pool_region(pool, j, &region_bytes);
        if (!regions[j] || !pool_slots ||
            pf_hip_pool_region_plan(l->gguf_type, l->k_storage, l->n_out, pool_slots, &want_bytes, &file_bytes, &expert_bytes[j],
                                    &scale_offsets[j]) ||
            /* a pool that was not told its formats holds file bytes: right only where the kernels read those */
            (format == UINT32_MAX ? scale_offsets[j] != 0 : format != l->gguf_type) || file_bytes != l->expert_bytes ||
            region_bytes < want_bytes)
            return moe_status(err, QW4_SHAPE, "the pool's slots do not hold this layer's experts");
    }
    uint32_t *ids = malloc(pairs * 2 * sizeof *ids), *slots = ids ? ids + pairs : NULL, word = 0;
    if (!ids) return moe_status(err, QW4_OOM, "streaming staging");
    Qwen4Status st = QW4_OK;
    int rc = pf_hip_moe_route_streamed_host(m->device, w->device, x.data, x.stride_bytes[0], T, tiled_mask, ids, &word);
    if (rc) st = pf_device_status(rc, err, "qwen4_moe");
    else if (word & PF_HIP_ERR_NONFINITE) st = moe_status(err, QW4_NONFINITE, "nonfinite value in the MoE block");
    else if (word) st = moe_status(err, QW4_GPU_ERROR, "device error word");
    else if (qw4_pool_acquire(pool, layer, ids, pairs, slots))
        st = moe_status(err, QW4_IO, "expert pool: every slot pinned, or a read of the model file failed");
    if (!st) {
        rc = pf_hip_moe_experts_streamed_host(m->device, w->device, regions, expert_bytes, scale_offsets, (uint32_t)pool_slots, tiled_mask, slots, y.data,
                                              y.stride_bytes[0], routes ? routes->ids.data : NULL,
                                              routes ? routes->ids.row_stride_bytes : 0,
                                              routes ? routes->weights.data : NULL,
                                              routes ? routes->weights.stride_bytes[0] : 0, T, &word);
        qw4_pool_release(pool, slots, pairs);
        if (rc) st = pf_device_status(rc, err, "qwen4_moe");
        else if (word & PF_HIP_ERR_NONFINITE) st = moe_status(err, QW4_NONFINITE, "nonfinite value in the MoE block");
        else if (word) st = moe_status(err, QW4_GPU_ERROR, "device error word");
        else st = moe_status(err, QW4_OK, "");
    }
    free(ids);
    return st;
}

static Qwen4Status forward_checked(const Qwen4Moe *m, QW4ExpertPool *pool, uint32_t layer, Qwen4F32 x, Qwen4F32Mut y,
                                   Qwen4MoeRoutes *routes, Qwen4MoeWork *w, Qwen4Error *err) {
    if (!m || !w) return moe_status(err, QW4_INVALID_ARGUMENT, "null forward handle");
    if (w->owner != m) return moe_status(err, QW4_OWNER, "workspace belongs to another MoE");
    if (!m->alive || w->failed) return moe_status(err, QW4_BAD_STATE, "inactive MoE/workspace; reset required");
    if (w->busy) return moe_status(err, QW4_BUSY, "workspace executing");
    if (m->streamed != (pool != NULL))
        return moe_status(err, QW4_BAD_STATE, m->streamed ? "a streamed layer forwards through an expert pool"
                                                           : "the layer's experts are resident: no pool applies");
    if (m->streamed && w->observer) return moe_status(err, QW4_BAD_STATE, "the observer needs the host weight bytes");
    const size_t T = x.dim[0], H = m->cfg.hidden_size, K = m->cfg.top_k;
    if (T > w->cap) return moe_status(err, QW4_CAPACITY, "batch exceeds token capacity");
    Range r[4];
    size_t nr = 2;
    TRY(RANGE_F32(x, T, H, &r[0]));
    TRY(RANGE_F32(y, T, H, &r[1]));
    if (routes) {
        TRY(RANGE_F32(routes->weights, T, K, &r[2]));
        if (routes->ids.rows != T || routes->ids.cols != K)
            return moe_status(err, QW4_SHAPE, "optional route shape mismatch");
        TRY(range_rows(routes->ids.data, routes->ids.capacity_bytes, T, K, routes->ids.row_stride_bytes, &r[3], err));
        nr = 4;
    }
    TRY(all_disjoint(r, nr, err));
    for (size_t a = 0; a < 8 && m->host_spans; a++) {
        const Range wr = {(uintptr_t)m->w[a].span.data, (uintptr_t)m->w[a].span.data + m->w[a].layout.tensor_bytes};
        for (size_t b = 0; b < nr; b++) {
            const Range two[2] = {r[b], wr};
            TRY(all_disjoint(two, 2, err));
        }
    }
    const size_t xs = x.stride_bytes[0] / 4;
    for (size_t row = 0; row < T; row++)
        for (size_t col = 0; col < H; col++)
            if (!isfinite(x.data[row * xs + col])) return moe_status(err, QW4_NONFINITE, "nonfinite input");
    if (!T) return moe_status(err, QW4_OK, "");
    /* the routing trace needs the ids also when the caller did not ask for them */
    Qwen4MoeRoutes traced;
    void *trace_memory = NULL;
    if (m->route_log && !routes) {
        trace_memory = malloc(T * K * 8);
        if (!trace_memory) return moe_status(err, QW4_OOM, "route log staging");
        traced = (Qwen4MoeRoutes){{trace_memory, T * K * 4, T, K, K * 4}, rows_of((float *)trace_memory + T * K, T, K)};
        routes = &traced;
    }
    w->busy = true;
    Qwen4Status st;
    if (w->observer) st = observed_forward(w, x, y, routes, err);
    else if (pool) st = streamed_forward(m, w, pool, layer, x, y, routes, err);
    else {
        uint32_t word = 0;
        int rc = pf_hip_moe_forward_host(m->device, w->device, x.data, x.stride_bytes[0], y.data, y.stride_bytes[0],
                                         routes ? routes->ids.data : NULL, routes ? routes->ids.row_stride_bytes : 0,
                                         routes ? routes->weights.data : NULL,
                                         routes ? routes->weights.stride_bytes[0] : 0, T, &word);
        if (rc) st = pf_device_status(rc, err, "qwen4_moe");
        else if (word & PF_HIP_ERR_NONFINITE) st = moe_status(err, QW4_NONFINITE, "nonfinite value in the MoE block");
        else if (word) st = moe_status(err, QW4_GPU_ERROR, "device error word");
        else st = moe_status(err, QW4_OK, "");
    }
    w->busy = false;
    if (st) w->failed = true;
    else if (m->route_log) route_log_append((Qwen4Moe *)m, routes->ids.data, routes->ids.row_stride_bytes / 4, T);
    free(trace_memory);
    return st;
}

Qwen4Status qwen4_moe_forward(const Qwen4Moe *m, Qwen4F32 x, Qwen4F32Mut y, Qwen4MoeRoutes *routes, Qwen4MoeWork *w,
                              Qwen4Error *err) {
    return forward_checked(m, NULL, 0, x, y, routes, w, err);
}

Qwen4Status pf_moe_forward_streamed(const Qwen4Moe *m, QW4ExpertPool *pool, uint32_t layer, Qwen4F32 x, Qwen4F32Mut y,
                                    Qwen4MoeRoutes *routes, Qwen4MoeWork *w, Qwen4Error *err) {
    if (!pool) return moe_status(err, QW4_INVALID_ARGUMENT, "null expert pool");
    return forward_checked(m, pool, layer, x, y, routes, w, err);
}

/* ---- the block between its two hyper-connection steps (src/qwen4_forward.c:362-367) ------------
 * Validation in the order of the three calls it stands for: the read's views, the forward's
 * handles and routes, the add's views.  The arithmetic and the finite checks run on the device;
 * the residual is written back only when the error word stayed clear. */
Qwen4Status pf_moe_forward_hc(const Qwen4Moe *m, const Qwen4HcShape *s, Qwen4F32 normed, Qwen4F32 logits,
                              Qwen4F32Mut residual, Qwen4F32 inject, Qwen4MoeRoutes *routes, Qwen4MoeWork *w,
                              Qwen4Error *err) {
    TRY(pf_hc_admit_shape(s, err));
    size_t span[2], rspan;
    TRY(pf_hc_admit_read_inputs(s, normed, logits, span, err));
    if (!m || !w) return moe_status(err, QW4_INVALID_ARGUMENT, "null forward handle");
    if (w->owner != m) return moe_status(err, QW4_OWNER, "workspace belongs to another MoE");
    if (!m->alive || w->failed) return moe_status(err, QW4_BAD_STATE, "inactive MoE/workspace; reset required");
    if (w->busy) return moe_status(err, QW4_BUSY, "workspace executing");
    const size_t T = normed.dim[0], H = m->cfg.hidden_size, K = m->cfg.top_k;
    if (s->hidden_size != H) return moe_status(err, QW4_SHAPE, "HC hidden size differs from the MoE's");
    if (T > w->cap) return moe_status(err, QW4_CAPACITY, "batch exceeds token capacity");
    Range r[5];
    size_t nr = 0;
    if (routes) {
        TRY(RANGE_F32(routes->weights, T, K, &r[0]));
        if (routes->ids.rows != T || routes->ids.cols != K)
            return moe_status(err, QW4_SHAPE, "optional route shape mismatch");
        TRY(range_rows(routes->ids.data, routes->ids.capacity_bytes, T, K, routes->ids.row_stride_bytes, &r[1], err));
        nr = 2;
    }
    if (residual.dim[0] != T) return moe_status(err, QW4_SHAPE, "residual token count differs from the input's");
    TRY(pf_hc_admit_add(s, residual, NULL, 0, inject, &rspan, err));
    r[nr++] = (Range){(uintptr_t)residual.data, (uintptr_t)residual.data + rspan};
    r[nr++] = (Range){(uintptr_t)normed.data, (uintptr_t)normed.data + span[0]};
    r[nr++] = (Range){(uintptr_t)logits.data, (uintptr_t)logits.data + span[1]};
    /* outputs (routes, residual) may not overlap each other or any input; the two read inputs may
     * share memory with each other, as they may for qwen4_hc_read */
    for (size_t i = 0; i + 2 < nr; i++)
        for (size_t j = i + 1; j < nr; j++)
            if (r[i].lo < r[j].hi && r[j].lo < r[i].hi)
                return moe_status(err, QW4_INVALID_ARGUMENT, "overlapping views");
    if (!T) return moe_status(err, QW4_OK, "");
    Qwen4MoeRoutes traced;
    void *trace_memory = NULL;
    if (m->route_log && !routes) {
        trace_memory = malloc(T * K * 8);
        if (!trace_memory) return moe_status(err, QW4_OOM, "route log staging");
        traced = (Qwen4MoeRoutes){{trace_memory, T * K * 4, T, K, K * 4}, rows_of((float *)trace_memory + T * K, T, K)};
        routes = &traced;
    }
    w->busy = true;
    uint32_t word = 0;
    int rc = pf_hip_moe_forward_hc_host(m->device, w->device, normed.data, normed.stride_bytes[0],
                                        normed.stride_bytes[1], logits.data, logits.stride_bytes[0],
                                        logits.stride_bytes[1], residual.data, residual.stride_bytes[0],
                                        residual.stride_bytes[1], inject.data, inject.stride_bytes[0], s->streams, T,
                                        routes ? routes->ids.data : NULL, routes ? routes->ids.row_stride_bytes : 0,
                                        routes ? routes->weights.data : NULL,
                                        routes ? routes->weights.stride_bytes[0] : 0, &word);
    w->busy = false;
    if (!rc && !word && m->route_log) route_log_append((Qwen4Moe *)m, routes->ids.data, routes->ids.row_stride_bytes / 4, T);
    free(trace_memory);
    if (rc || word) {
        w->failed = true;
        if (rc) return pf_device_status(rc, err, "qwen4_moe");
        if (word & PF_HIP_ERR_NONFINITE)
            return moe_status(err, QW4_NONFINITE, "nonfinite value in the hyper-connection steps or the MoE block");
        return moe_status(err, QW4_GPU_ERROR, "device error word");
    }
    return moe_status(err, QW4_OK, "");
}
