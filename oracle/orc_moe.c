/* Oracle, MoE part: TEST INFRASTRUCTURE, never linked into the product.
 * Follows src/qwen4_moe.c; operation order and check order are the reference's. */
#include "orc.h"
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

typedef struct { uintptr_t lo, hi; } Extent;

/* arena buffers, src/qwen4_moe.c:10-11 */
enum { B_LOGITS, B_PROBS, B_SCORES, B_IDS, B_GATHER, B_DOWN, B_GATE, B_UP, B_ACT, B_SHARED, B_SG, B_SA,
       B_OFFSETS, B_CURSORS, B_P2R, B_R2P, B_COUNT };

struct OrcMoe {
    Qwen4MoeConfig cfg;
    QW4PackedCpuView w[8];
    size_t refs;
    bool alive;
};

struct OrcMoeWork {
    OrcMoe *owner;
    size_t cap, micro, bytes, size[B_COUNT];
    void *buf[B_COUNT], *arena;
    bool busy, failed;
    QW4MoeObserver observer;
    void *observer_ctx;
};

static Qwen4Status fail(Qwen4Error *err, Qwen4Status code, const char *detail) {
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
#define CHECK(expr) do { Qwen4Status s_ = (expr); if (s_ != QW4_OK) return s_; } while (0)

/* src/qwen4_moe.c:34-41 */
static Qwen4Status check_config(const Qwen4MoeConfig *c, Qwen4Error *err) {
    if (!c) return fail(err, QW4_INVALID_ARGUMENT, "null config");
    if (c->hidden_size == 0 || c->experts == 0 || c->top_k == 0 || c->top_k > c->experts ||
        c->intermediate == 0 || c->shared_intermediate == 0 || c->down_physical < c->intermediate)
        return fail(err, QW4_RANGE, "invalid MoE dimensions");
    return QW4_OK;
}

static Qwen4F32Mut dense(float *p, size_t rows, size_t cols) {
    Qwen4F32Mut v;
    memset(&v, 0, sizeof v);
    v.data = p; v.capacity_bytes = rows * cols * 4; v.rank = 2;
    v.dim[0] = rows; v.dim[1] = cols; v.dim[2] = 1; v.dim[3] = 1;
    v.stride_bytes[0] = cols * 4; v.stride_bytes[1] = 4;
    return v;
}
static Qwen4F32 ro(Qwen4F32Mut v) {
    Qwen4F32 r;
    memset(&r, 0, sizeof r);
    r.data = v.data; r.capacity_bytes = v.capacity_bytes; r.rank = v.rank;
    memcpy(r.dim, v.dim, sizeof r.dim);
    memcpy(r.stride_bytes, v.stride_bytes, sizeof r.stride_bytes);
    return r;
}

/* src/qwen4_moe.c:47-76 */
Qwen4Status orc_moe_create(const Qwen4MoeConfig *c, const Qwen4MoeWeights *weights, OrcMoe **out,
                           Qwen4Error *err) {
    if (out) *out = NULL;
    if (!out || !weights) return fail(err, QW4_INVALID_ARGUMENT, "null create argument");
    CHECK(check_config(c, err));
    QW4PackedCpuView w[8] = {weights->router, weights->gate, weights->up, weights->down,
                             weights->shared_gate, weights->shared_up, weights->shared_down,
                             weights->shared_router};
    size_t h = c->hidden_size, i = c->intermediate, s = c->shared_intermediate;
    size_t k_in[8] = {h, h, h, i, h, h, s, h}, n_out[8] = {c->experts, i, i, h, s, s, h, 1};
    for (size_t a = 0; a < 8; a++) {
        const QW4PackedLayout *l = &w[a].layout;
        size_t experts = (a >= 1 && a <= 3) ? c->experts : 1;
        size_t storage = a == 3 ? c->down_physical : k_in[a];
        if (l->k_logical != k_in[a] || l->n_out != n_out[a] || l->n_experts != experts ||
            l->k_storage != storage)
            return fail(err, QW4_SHAPE, "MoE weight shape mismatch");
        if ((a == 0 || a == 7) && l->gguf_type != 0) return fail(err, QW4_FORMAT, "router must be F32");
        /* an empty product validates descriptor and span without reading bytes */
        Qwen4F32Mut y0 = dense(NULL, 0, n_out[a]);
        Qwen4F32 x0 = ro(dense(NULL, 0, k_in[a]));
        CHECK(orc_packed_matmul(&w[a], 0, x0, y0, err));
    }
    OrcMoe *m = calloc(1, sizeof *m);
    if (!m) return fail(err, QW4_OOM, "MoE allocation");
    m->cfg = *c;
    memcpy(m->w, w, sizeof w);
    m->refs = 1;
    m->alive = true;
    *out = m;
    return fail(err, QW4_OK, "");
}

static void release(OrcMoe *m) { if (m && --m->refs == 0) free(m); }
void orc_moe_destroy(OrcMoe *m) { if (m && m->alive) { m->alive = false; release(m); } }

/* src/qwen4_moe.c:80-104: sixteen buffers for min(cap, 32) tokens, 8-byte rounded */
static Qwen4Status plan(const OrcMoe *m, size_t cap, OrcMoeWork *p, Qwen4Error *err) {
    if (!m || !m->alive) return fail(err, QW4_BAD_STATE, "inactive MoE");
    size_t t = cap < 32 ? cap : 32, k = m->cfg.top_k, e = m->cfg.experts, h = m->cfg.hidden_size;
    size_t i = m->cfg.intermediate > m->cfg.shared_intermediate ? m->cfg.intermediate
                                                                : m->cfg.shared_intermediate;
    if (k && t > SIZE_MAX / k) return fail(err, QW4_OVERFLOW, "pair count overflow");
    size_t pairs = t * k;
    size_t rows[B_COUNT] = {t, t, t, t, pairs, pairs, t, t, t, t, t, t, e + 1, e, pairs, pairs};
    size_t cols[B_COUNT] = {e, e, k, k, h, h, i, i, i, h, 1, 1, 1, 1, 1, 1};
    p->bytes = 0; p->cap = cap; p->micro = t;
    for (size_t j = 0; j < B_COUNT; j++) {
        size_t unit = j < B_OFFSETS ? 4 : sizeof(size_t);
        if (rows[j] > SIZE_MAX / cols[j] || rows[j] * cols[j] > (SIZE_MAX - 7) / unit)
            return fail(err, QW4_OVERFLOW, "scratch size overflow");
        size_t bytes = (rows[j] * cols[j] * unit + 7) & ~(size_t)7;
        if (p->bytes > SIZE_MAX - bytes) return fail(err, QW4_OVERFLOW, "arena overflow");
        p->size[j] = bytes;
        p->bytes += bytes;
    }
    if (p->bytes > SIZE_MAX - sizeof *p) return fail(err, QW4_OVERFLOW, "workspace overflow");
    return QW4_OK;
}

Qwen4Status orc_moe_work_size(const OrcMoe *m, size_t cap, size_t *bytes, Qwen4Error *err) {
    if (!bytes) return fail(err, QW4_INVALID_ARGUMENT, "null size output");
    *bytes = 0;
    OrcMoeWork p;
    memset(&p, 0, sizeof p);
    CHECK(plan(m, cap, &p, err));
    *bytes = sizeof p + p.bytes;
    return fail(err, QW4_OK, "");
}

Qwen4Status orc_moe_work_create(const OrcMoe *m, size_t cap, size_t budget, OrcMoeWork **out,
                                Qwen4Error *err) {
    if (out) *out = NULL;
    if (!out) return fail(err, QW4_INVALID_ARGUMENT, "null workspace output");
    OrcMoeWork p;
    memset(&p, 0, sizeof p);
    CHECK(plan(m, cap, &p, err));
    if (budget < sizeof p + p.bytes) return fail(err, QW4_CAPACITY, "workspace budget too small");
    OrcMoeWork *w = malloc(sizeof *w);
    if (!w) return fail(err, QW4_OOM, "workspace metadata");
    *w = p;
    w->arena = calloc(1, p.bytes ? p.bytes : 1);
    if (!w->arena) { free(w); return fail(err, QW4_OOM, "workspace arena"); }
    size_t off = 0;
    for (size_t j = 0; j < B_COUNT; j++) { w->buf[j] = (char *)w->arena + off; off += w->size[j]; }
    w->owner = (OrcMoe *)m;
    w->owner->refs++;
    *out = w;
    return fail(err, QW4_OK, "");
}

Qwen4Status orc_moe_work_reset(OrcMoeWork *w, Qwen4Error *err) {
    if (!w) return fail(err, QW4_INVALID_ARGUMENT, "null workspace");
    if (w->busy) return fail(err, QW4_BUSY, "workspace executing");
    if (!w->owner->alive) return fail(err, QW4_BAD_STATE, "destroyed owner");
    memset(w->arena, 0, w->bytes);
    w->failed = false;
    return fail(err, QW4_OK, "");
}

void orc_moe_work_destroy(OrcMoeWork *w) {
    if (w && !w->busy) { release(w->owner); free(w->arena); free(w); }
}

void orc_moe_observe(OrcMoeWork *w, QW4MoeObserver fn, void *ctx) {
    if (w && !w->busy) { w->observer = fn; w->observer_ctx = ctx; }
}

/* src/qwen4_moe.c:134-148 */
static Qwen4Status extent_of(const void *data, size_t cap, size_t bytes, size_t alignment, Extent *x,
                             Qwen4Error *err) {
    x->lo = x->hi = 0;
    if (bytes == 0) return QW4_OK;
    if (cap < bytes) return fail(err, QW4_CAPACITY, "view capacity too small");
    if (!data) return fail(err, QW4_INVALID_ARGUMENT, "null nonempty view");
    uintptr_t lo = (uintptr_t)data;
    if (lo % alignment) return fail(err, QW4_STRIDE, "unaligned view");
    if (bytes > UINTPTR_MAX - lo) return fail(err, QW4_OVERFLOW, "address extent overflow");
    x->lo = lo; x->hi = lo + bytes;
    return QW4_OK;
}

/* src/qwen4_moe.c:152-165: the bounding extent includes the row padding */
static Qwen4Status extent_rows(const void *data, size_t cap, size_t rows, size_t cols, size_t pitch,
                               Extent *x, Qwen4Error *err) {
    x->lo = x->hi = 0;
    if (cols > SIZE_MAX / 4) return fail(err, QW4_OVERFLOW, "row bytes overflow");
    size_t row_bytes = cols * 4;
    if (pitch % 4 || pitch < row_bytes)
        return fail(err, QW4_STRIDE, "row stride must cover contiguous features");
    if (rows == 0) return QW4_OK;
    if (rows - 1 > (SIZE_MAX - row_bytes) / pitch) return fail(err, QW4_OVERFLOW, "view extent overflow");
    return extent_of(data, cap, (rows - 1) * pitch + row_bytes, 4, x, err);
}

/* src/qwen4_moe.c:167-174 */
static Qwen4Status extent_f32(Qwen4F32 v, size_t rows, size_t cols, Extent *x, Qwen4Error *err) {
    if (v.rank != 2 || v.dim[0] != rows || v.dim[1] != cols)
        return fail(err, QW4_SHAPE, "expected rank-2 token-major view");
    if (v.stride_bytes[1] != sizeof(float)) return fail(err, QW4_STRIDE, "features must be contiguous");
    return extent_rows(v.data, v.capacity_bytes, rows, cols, v.stride_bytes[0], x, err);
}

/* src/qwen4_moe.c:180-186 */
static Qwen4Status check_disjoint(const Extent *x, size_t n, Qwen4Error *err) {
    for (size_t i = 0; i < n; i++)
        for (size_t j = 0; j < i; j++)
            if (x[i].lo < x[j].hi && x[j].lo < x[i].hi)
                return fail(err, QW4_INVALID_ARGUMENT, "overlapping views");
    return QW4_OK;
}

/* src/qwen4_moe.c:188-249 */
Qwen4Status orc_moe_route(const Qwen4MoeConfig *c, Qwen4F32 logits, Qwen4MoeRoutes routes,
                          Qwen4F32Mut probabilities, Qwen4Error *err) {
    CHECK(check_config(c, err));
    const size_t T = logits.dim[0], E = c->experts, K = c->top_k;
    Extent x[4];
    CHECK(extent_f32(logits, T, E, &x[0], err));
    CHECK(extent_f32(ro(probabilities), T, E, &x[1], err));
    CHECK(extent_f32(ro(routes.weights), T, K, &x[2], err));
    if (routes.ids.rows != T || routes.ids.cols != K) return fail(err, QW4_SHAPE, "route ID shape mismatch");
    CHECK(extent_rows(routes.ids.data, routes.ids.capacity_bytes, T, K, routes.ids.row_stride_bytes, &x[3],
                      err));
    CHECK(check_disjoint(x, 4, err));
    const size_t zs = logits.stride_bytes[0] / 4, ps = probabilities.stride_bytes[0] / 4;
    const size_t ws = routes.weights.stride_bytes[0] / 4, is = routes.ids.row_stride_bytes / 4;
    for (size_t t = 0; t < T; t++)
        for (size_t e = 0; e < E; e++)
            if (!isfinite(logits.data[t * zs + e])) {
                Qwen4Status st = fail(err, QW4_NONFINITE, "nonfinite router logit");
                if (err) err->row = t;
                return st;
            }
    for (size_t t = 0; t < T; t++) {
        const float *z = logits.data + t * zs;
        float *p = probabilities.data + t * ps, *w = routes.weights.data + t * ws;
        uint32_t *ids = routes.ids.data + t * is;
        float top = z[0], sum = 0.0f;
        for (size_t e = 1; e < E; e++) if (z[e] > top) top = z[e];
        for (size_t e = 0; e < E; e++) { p[e] = expf(z[e] - top); sum += p[e]; }
        for (size_t e = 0; e < E; e++) p[e] /= sum;
        float chosen = 0.0f;
        for (size_t slot = 0; slot < K; slot++) {
            size_t best = 0;
            bool have = false;
            for (size_t e = 0; e < E; e++) {
                bool taken = false;
                for (size_t j = 0; j < slot; j++) taken |= ids[j] == e;
                if (!taken && (!have || p[e] > p[best])) { best = e; have = true; }
            }
            ids[slot] = (uint32_t)best;
            w[slot] = p[best];
            chosen += w[slot];
        }
        if (c->norm_topk_prob) for (size_t slot = 0; slot < K; slot++) w[slot] /= chosen;
    }
    return fail(err, QW4_OK, "");
}

/* src/qwen4_moe.c:251-303 */
Qwen4Status orc_moe_group_pairs(const Qwen4MoeConfig *c, Qwen4U32Mut ids, QW4MoeGrouping g, Qwen4Error *err) {
    CHECK(check_config(c, err));
    if (ids.cols != c->top_k) return fail(err, QW4_SHAPE, "group ID shape mismatch");
    const size_t E = c->experts, K = c->top_k;
    if (ids.rows > SIZE_MAX / K || E == SIZE_MAX) return fail(err, QW4_OVERFLOW, "group count overflow");
    const size_t pairs = ids.rows * K;
    Extent x[5];
    CHECK(extent_rows(ids.data, ids.capacity_bytes, ids.rows, ids.cols, ids.row_stride_bytes, &x[0], err));
    const void *ptr[4] = {g.offsets, g.cursors, g.pair_to_row, g.row_to_pair};
    const size_t count[4] = {E + 1, E, pairs, pairs};
    const size_t cap[4] = {g.offsets_capacity_bytes, g.cursors_capacity_bytes,
                           g.pair_to_row_capacity_bytes, g.row_to_pair_capacity_bytes};
    for (size_t a = 0; a < 4; a++) {
        if (count[a] > SIZE_MAX / sizeof(size_t)) return fail(err, QW4_OVERFLOW, "group array bytes overflow");
        CHECK(extent_of(ptr[a], cap[a], count[a] * sizeof(size_t), _Alignof(size_t), &x[a + 1], err));
    }
    CHECK(check_disjoint(x, 5, err));
    const size_t is = ids.row_stride_bytes / 4;
    for (size_t t = 0; t < ids.rows; t++)
        for (size_t s = 0; s < K; s++) {
            uint32_t e = ids.data[t * is + s];
            if (e >= E) return fail(err, QW4_RANGE, "expert ID out of range");
            for (size_t j = 0; j < s; j++)
                if (ids.data[t * is + j] == e) return fail(err, QW4_INVALID_ARGUMENT, "duplicate expert ID");
        }
    memset(g.offsets, 0, (E + 1) * sizeof(size_t));
    for (size_t t = 0; t < ids.rows; t++)
        for (size_t s = 0; s < K; s++) g.offsets[ids.data[t * is + s] + 1]++;
    for (size_t e = 0; e < E; e++) { g.offsets[e + 1] += g.offsets[e]; g.cursors[e] = g.offsets[e]; }
    for (size_t t = 0; t < ids.rows; t++)
        for (size_t s = 0; s < K; s++) {
            size_t pair = t * K + s, row = g.cursors[ids.data[t * is + s]]++;
            g.pair_to_row[pair] = row;
            g.row_to_pair[row] = pair;
        }
    return fail(err, QW4_OK, "");
}

static void trace(OrcMoeWork *w, size_t stage, size_t expert, size_t token, Qwen4F32 in, Qwen4F32Mut out) {
    if (w->observer) w->observer(w->observer_ctx, stage, expert, token, in, ro(out));
}

static Qwen4Status linear(OrcMoeWork *w, size_t stage, size_t expert, size_t token, Qwen4F32 x, Qwen4F32Mut y,
                          Qwen4Error *err) {
    Qwen4Status st = orc_packed_matmul(&w->owner->w[stage], expert, x, y, err);
    if (st == QW4_OK) trace(w, stage, expert, token, x, y);
    return st;
}

/* src/qwen4_moe.c:318-333: gate, up, SiLU(gate), product with finite check, down */
static Qwen4Status expert_block(OrcMoeWork *w, size_t expert, size_t token, Qwen4F32 x, Qwen4F32Mut y,
                                bool shared, Qwen4Error *err) {
    const Qwen4MoeConfig *c = &w->owner->cfg;
    size_t n = x.dim[0], i = shared ? c->shared_intermediate : c->intermediate;
    Qwen4F32Mut g = dense(w->buf[B_GATE], n, i), u = dense(w->buf[B_UP], n, i), a = dense(w->buf[B_ACT], n, i);
    CHECK(linear(w, shared ? 4 : 1, expert, token, x, g, err));
    CHECK(linear(w, shared ? 5 : 2, expert, token, x, u, err));
    CHECK(orc_activate(1, ro(g), a, err));
    trace(w, 8, shared ? SIZE_MAX : expert, token, ro(g), a);
    for (size_t j = 0; j < n * i; j++) {
        a.data[j] *= u.data[j];
        if (!isfinite(a.data[j])) return fail(err, QW4_NONFINITE, "gate/up overflow");
    }
    trace(w, 9, shared ? SIZE_MAX : expert, token, ro(u), a);
    return linear(w, shared ? 6 : 3, expert, token, ro(a), y, err);
}

/* src/qwen4_moe.c:334-382 */
static Qwen4Status batch(OrcMoeWork *w, Qwen4F32 x, Qwen4F32Mut y, size_t token, Qwen4Error *err) {
    const Qwen4MoeConfig *c = &w->owner->cfg;
    const size_t T = x.dim[0], E = c->experts, K = c->top_k, H = c->hidden_size, pairs = T * K;
    Qwen4F32Mut z = dense(w->buf[B_LOGITS], T, E), p = dense(w->buf[B_PROBS], T, E);
    Qwen4MoeRoutes r;
    r.ids.data = w->buf[B_IDS]; r.ids.capacity_bytes = T * K * 4; r.ids.rows = T; r.ids.cols = K;
    r.ids.row_stride_bytes = K * 4;
    r.weights = dense(w->buf[B_SCORES], T, K);
    CHECK(linear(w, 0, 0, token, x, z, err));
    CHECK(orc_moe_route(c, ro(z), r, p, err));
    QW4MoeGrouping g = {w->buf[B_OFFSETS], w->size[B_OFFSETS], w->buf[B_CURSORS], w->size[B_CURSORS],
                        w->buf[B_P2R], w->buf[B_R2P], w->size[B_P2R], w->size[B_R2P]};
    CHECK(orc_moe_group_pairs(c, r.ids, g, err));
    float *gather = w->buf[B_GATHER], *down = w->buf[B_DOWN];
    const size_t xs = x.stride_bytes[0] / 4, ys = y.stride_bytes[0] / 4;
    for (size_t row = 0; row < pairs; row++)
        memcpy(gather + row * H, x.data + (g.row_to_pair[row] / K) * xs, H * 4);
    for (size_t e = 0; e < E; e++) {
        size_t first = g.offsets[e], n = g.offsets[e + 1] - first;
        if (n == 0) continue;
        CHECK(expert_block(w, e, token, ro(dense(gather + first * H, n, H)), dense(down + first * H, n, H),
                           false, err));
    }
    Qwen4F32Mut shared = dense(w->buf[B_SHARED], T, H);
    CHECK(expert_block(w, 0, token, x, shared, true, err));
    Qwen4F32Mut sg = dense(w->buf[B_SG], T, 1), sa = dense(w->buf[B_SA], T, 1);
    CHECK(linear(w, 7, 0, token, x, sg, err));
    CHECK(orc_activate(0, ro(sg), sa, err));
    trace(w, 10, SIZE_MAX, token, ro(sg), sa);
    for (size_t row = 0; row < T; row++)
        for (size_t col = 0; col < H; col++) {
            float sum = 0;
            for (size_t slot = 0; slot < K; slot++) {
                size_t pair = row * K + slot;
                float term = r.weights.data[pair] * down[g.pair_to_row[pair] * H + col];
                sum += term;
                if (!isfinite(term) || !isfinite(sum)) return fail(err, QW4_NONFINITE, "routed reduction overflow");
            }
            y.data[row * ys + col] = sum;
        }
    trace(w, 11, SIZE_MAX, token, x, y);
    for (size_t row = 0; row < T; row++)
        for (size_t col = 0; col < H; col++) {
            float term = sa.data[row] * shared.data[row * H + col];
            float *o = y.data + row * ys + col;
            *o += term;
            if (!isfinite(term) || !isfinite(*o)) return fail(err, QW4_NONFINITE, "shared sum overflow");
        }
    trace(w, 12, SIZE_MAX, token, x, y);
    return QW4_OK;
}

/* src/qwen4_moe.c:384-431 */
Qwen4Status orc_moe_forward(const OrcMoe *m, Qwen4F32 x, Qwen4F32Mut y, Qwen4MoeRoutes *routes, OrcMoeWork *w,
                            Qwen4Error *err) {
    if (!m || !w) return fail(err, QW4_INVALID_ARGUMENT, "null forward handle");
    if (w->owner != m) return fail(err, QW4_OWNER, "workspace belongs to another MoE");
    if (!m->alive || w->failed) return fail(err, QW4_BAD_STATE, "inactive MoE/workspace; reset required");
    if (w->busy) return fail(err, QW4_BUSY, "workspace executing");
    const size_t T = x.dim[0], H = m->cfg.hidden_size, K = m->cfg.top_k;
    if (T > w->cap) return fail(err, QW4_CAPACITY, "batch exceeds token capacity");
    Extent v[4];
    size_t nv = 2;
    CHECK(extent_f32(x, T, H, &v[0], err));
    CHECK(extent_f32(ro(y), T, H, &v[1], err));
    if (routes) {
        CHECK(extent_f32(ro(routes->weights), T, K, &v[2], err));
        if (routes->ids.rows != T || routes->ids.cols != K)
            return fail(err, QW4_SHAPE, "optional route shape mismatch");
        CHECK(extent_rows(routes->ids.data, routes->ids.capacity_bytes, T, K, routes->ids.row_stride_bytes,
                          &v[3], err));
        nv = 4;
    }
    CHECK(check_disjoint(v, nv, err));
    for (size_t a = 0; a < 8; a++) {
        Extent wx = {(uintptr_t)m->w[a].span.data, (uintptr_t)m->w[a].span.data + m->w[a].layout.tensor_bytes};
        for (size_t b = 0; b < nv; b++) {
            Extent two[2] = {v[b], wx};
            CHECK(check_disjoint(two, 2, err));
        }
    }
    const size_t xs = x.stride_bytes[0] / 4;
    for (size_t row = 0; row < T; row++)
        for (size_t col = 0; col < H; col++)
            if (!isfinite(x.data[row * xs + col])) return fail(err, QW4_NONFINITE, "nonfinite input");
    w->busy = true;
    for (size_t start = 0; start < T;) {
        size_t n = T - start < w->micro ? T - start : w->micro;
        Qwen4F32 bx = x;
        Qwen4F32Mut by = y;
        bx.data += start * xs; bx.capacity_bytes -= start * x.stride_bytes[0]; bx.dim[0] = n;
        by.data += start * (y.stride_bytes[0] / 4); by.capacity_bytes -= start * y.stride_bytes[0]; by.dim[0] = n;
        Qwen4Status st = batch(w, bx, by, start, err);
        if (st != QW4_OK) { w->busy = false; w->failed = true; return st; }
        if (routes)
            for (size_t row = 0; row < n; row++) {
                memcpy(routes->ids.data + (start + row) * (routes->ids.row_stride_bytes / 4),
                       (uint32_t *)w->buf[B_IDS] + row * K, K * 4);
                memcpy(routes->weights.data + (start + row) * (routes->weights.stride_bytes[0] / 4),
                       (float *)w->buf[B_SCORES] + row * K, K * 4);
            }
        start += n;
    }
    w->busy = false;
    return fail(err, QW4_OK, "");
}
