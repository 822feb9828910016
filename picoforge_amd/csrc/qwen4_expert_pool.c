/* Expert pool in device memory (include/qwen4_expert_pool.h): the bookkeeping of
 * src/qwen4_expert_pool.c of the reference restated for HBM-resident slots.
 *
 * Recency is a counter stamped on a slot whenever it is acquired; the victim of a miss is the slot
 * with the oldest stamp among those nobody pins (fresh pools stamp slot s with s, so slot 0 goes first,
 * as in the reference).  A scan over the slots per miss is enough: pools hold a few thousand slots and
 * a miss costs a file read of megabytes.  The readers are threads the pool starts once, at its first miss, each
 * with a stage of its own (page-locked host memory, device memory and a stream, pf_hip_stage_create): a reader
 * preads one matrix of one missed expert into its page-locked memory and has it copied (split, tiled) into the
 * slot on its stream, so no acquire starts a thread or allocates anything. */
#define _GNU_SOURCE
#include "../../include/qwen4_expert_pool.h"
#include "../../include/pf_moe_hip.h"
#include <pthread.h>
#include <stdatomic.h>
#include <stdbool.h>
#include <stdlib.h>
#include <time.h>
#include <unistd.h>

#define NO_SLOT UINT32_MAX
#define QW4_POOL_MAX_READERS 64

struct QW4ExpertPool {
    int fd;
    uint32_t n_layers, experts, slots, readers;
    size_t bytes[3], region_bytes[3];
    QW4ExpertLayer *layers;
    void *region[3];        /* device memory: slots * bytes[m] each */
    uint32_t *where;        /* [layer * experts + expert] -> slot or NO_SLOT */
    uint32_t *holds;        /* [slot] -> layer * experts + expert or NO_SLOT */
    uint32_t *pins;         /* [slot] */
    uint64_t *stamp, clock; /* [slot] recency */
    uint32_t *new_slot, *new_expert;   /* the misses of the acquire in progress */
    QW4PoolStats stats;
    /* pf_pool_set_formats: slots in the device layout */
    bool formatted, used;
    uint32_t type[3];
    size_t k_storage[3], n_out[3], scale_offset[3];
    /* the readers: started at the first miss; they sleep on `wake` between acquires */
    pthread_mutex_t lock;
    pthread_cond_t wake, done;
    pthread_t thread[QW4_POOL_MAX_READERS];
    PfHipStage *stage[QW4_POOL_MAX_READERS + 1];   /* the last one is the acquiring thread's own */
    uint32_t started;
    uint64_t round;            /* incremented per batch of reads; a reader takes part once per round */
    uint32_t running;          /* readers still at work on the current round */
    bool quit, lock_ready;
    struct Reads *reads;       /* the current round's */
};

QW4ExpertPool *qw4_pool_create(int fd, const QW4ExpertLayer *layers, uint32_t n_layers, uint32_t experts,
                               const size_t bytes[3], uint32_t slots) {
    if (fd < 0 || !layers || !bytes || !n_layers || !experts || !slots || slots == NO_SLOT) return NULL;
    if (!bytes[0] || !bytes[1] || !bytes[2] || (uint64_t)n_layers * experts >= NO_SLOT) return NULL;
    QW4ExpertPool *p = calloc(1, sizeof *p);
    if (!p) return NULL;
    p->fd = fd; p->n_layers = n_layers; p->experts = experts; p->slots = slots; p->readers = 8;
    if (pthread_mutex_init(&p->lock, NULL) || pthread_cond_init(&p->wake, NULL) || pthread_cond_init(&p->done, NULL)) { free(p); return NULL; }
    p->lock_ready = true;
    const size_t keys = (size_t)n_layers * experts;
    p->layers = malloc(n_layers * sizeof *p->layers);
    p->where = malloc(keys * sizeof *p->where);
    p->holds = malloc(slots * sizeof *p->holds);
    p->pins = calloc(slots, sizeof *p->pins);
    p->stamp = malloc(slots * sizeof *p->stamp);
    p->new_slot = malloc(slots * sizeof *p->new_slot);
    p->new_expert = malloc(slots * sizeof *p->new_expert);
    if (!p->layers || !p->where || !p->holds || !p->pins || !p->stamp || !p->new_slot || !p->new_expert) {
        qw4_pool_destroy(p);
        return NULL;
    }
    for (uint32_t l = 0; l < n_layers; l++) p->layers[l] = layers[l];
    for (size_t k = 0; k < keys; k++) p->where[k] = NO_SLOT;
    for (uint32_t s = 0; s < slots; s++) { p->holds[s] = NO_SLOT; p->stamp[s] = s; }
    p->clock = slots;
    for (int m = 0; m < 3; m++) {
        p->bytes[m] = bytes[m];
        p->region_bytes[m] = (size_t)slots * bytes[m];
        if (pf_hip_malloc(&p->region[m], p->region_bytes[m]) != PF_HIP_OK) {
            p->region[m] = NULL;
            qw4_pool_destroy(p);
            return NULL;
        }
    }
    return p;
}

void qw4_pool_destroy(QW4ExpertPool *p) {
    if (!p) return;
    if (p->lock_ready) {
        pthread_mutex_lock(&p->lock);
        p->quit = true;
        pthread_cond_broadcast(&p->wake);
        pthread_mutex_unlock(&p->lock);
        for (uint32_t j = 0; j < p->started; j++) pthread_join(p->thread[j], NULL);
        for (uint32_t j = 0; j <= QW4_POOL_MAX_READERS; j++) pf_hip_stage_destroy(p->stage[j]);
        pthread_cond_destroy(&p->wake); pthread_cond_destroy(&p->done); pthread_mutex_destroy(&p->lock);
    }
    for (int m = 0; m < 3; m++)
        if (p->region[m]) pf_hip_free(p->region[m]);
    free(p->layers); free(p->where); free(p->holds); free(p->pins); free(p->stamp); free(p->new_slot); free(p->new_expert);
    free(p);
}

/* Extension: the matrices' formats, so that a slot holds its expert in the layout the kernels read (formats the
 * device stores split are split on arrival).  Before the first acquire only; the regions are allocated again. */
int pf_pool_set_formats(QW4ExpertPool *p, const uint32_t gguf_type[3], const size_t k_storage[3], const size_t n_out[3]) {
    if (!p || p->used || !gguf_type || !k_storage || !n_out) return -1;
    size_t region_bytes[3], file_bytes, payload_bytes, scale_offset[3];
    for (int m = 0; m < 3; m++)
        if (pf_hip_pool_region_plan(gguf_type[m], k_storage[m], n_out[m], p->slots, &region_bytes[m], &file_bytes,
                                    &payload_bytes, &scale_offset[m]) != PF_HIP_OK || file_bytes != p->bytes[m])
            return -1;
    for (int m = 0; m < 3; m++) {
        void *region = NULL;
        if (pf_hip_malloc(&region, region_bytes[m]) != PF_HIP_OK) return -1;   /* earlier matrices keep their new regions: sizes only grow */
        pf_hip_free(p->region[m]);
        p->region[m] = region;
        p->region_bytes[m] = region_bytes[m];
        p->type[m] = gguf_type[m]; p->k_storage[m] = k_storage[m]; p->n_out[m] = n_out[m]; p->scale_offset[m] = scale_offset[m];
    }
    p->formatted = true;
    return 0;
}

uint32_t pf_pool_slots(const QW4ExpertPool *p) { return p ? p->slots : 0; }
size_t pf_pool_scale_offset(const QW4ExpertPool *p, int matrix) {
    return p && p->formatted && matrix >= 0 && matrix < 3 ? p->scale_offset[matrix] : 0;
}
/* The format matrix m's slots are laid out for; UINT32_MAX: as the file stores it, whatever the format. */
uint32_t pf_pool_format(const QW4ExpertPool *p, int matrix) {
    return p && p->formatted && matrix >= 0 && matrix < 3 ? p->type[matrix] : UINT32_MAX;
}

void qw4_pool_set_readers(QW4ExpertPool *p, uint32_t readers) {
    if (p) p->readers = readers ? readers : 1;
}

void qw4_pool_release(QW4ExpertPool *p, const uint32_t *slots, size_t n) {
    if (!p || !slots) return;
    for (size_t i = 0; i < n; i++)
        if (slots[i] < p->slots && p->pins[slots[i]]) p->pins[slots[i]]--;
}

void *qw4_pool_region(const QW4ExpertPool *p, int matrix, size_t *bytes) {
    if (!p || matrix < 0 || matrix > 2) return NULL;
    if (bytes) *bytes = p->region_bytes[matrix];
    return p->region[matrix];
}

QW4PoolStats qw4_pool_stats(const QW4ExpertPool *p) {
    QW4PoolStats none = {0, 0, 0, 0, 0};
    return p ? p->stats : none;
}

/* ---- the reads of one acquire ------------------------------------------------------------------
 * A job is one matrix of one missed expert; the readers take jobs from a shared counter until none
 * is left.  (The reference hands reader g the jobs g, g + width, ...; which reader reads what does
 * not show in the result.) */
typedef struct Reads {
    QW4ExpertPool *p;
    uint32_t layer, misses;
    atomic_size_t next;
    atomic_int failed;
} Reads;

static int read_exactly(int fd, unsigned char *dst, size_t bytes, uint64_t offset) {
    size_t done = 0;
    while (done < bytes) {
        const ssize_t got = pread(fd, dst + done, bytes - done, (off_t)(offset + done));
        if (got <= 0) return -1;
        done += (size_t)got;
    }
    return 0;
}

static size_t widest_matrix(const QW4ExpertPool *p) {
    size_t widest = p->bytes[0];
    for (int m = 1; m < 3; m++) widest = p->bytes[m] > widest ? p->bytes[m] : widest;
    return widest;
}

/* one reader's share of a round: jobs from the shared counter, through its stage */
static void read_jobs(Reads *r, PfHipStage *stage) {
    QW4ExpertPool *p = r->p;
    unsigned char *host = pf_hip_stage_host(stage);
    for (;;) {
        const size_t job = atomic_fetch_add(&r->next, 1);
        if (job >= (size_t)r->misses * 3 || atomic_load(&r->failed)) break;
        const size_t miss = job / 3;
        const int m = (int)(job % 3);
        const uint64_t from = p->layers[r->layer].offset[m] + (uint64_t)p->new_expert[miss] * p->bytes[m];
        int rc = read_exactly(p->fd, host, p->bytes[m], from);
        if (!rc)
            rc = pf_hip_pool_store_staged(stage, p->formatted ? p->type[m] : UINT32_MAX, p->k_storage[m], p->n_out[m], p->slots,
                                          p->region[m], p->new_slot[miss], p->bytes[m]);
        if (rc) atomic_store(&r->failed, 1);
    }
}

typedef struct { QW4ExpertPool *p; uint32_t index; uint64_t round; } ReaderArg;

static void *reader_main(void *arg) {
    ReaderArg *me = arg;
    QW4ExpertPool *p = me->p;
    const uint32_t index = me->index;
    uint64_t seen = me->round;   /* the rounds before this reader existed are not its business */
    free(me);
    pthread_mutex_lock(&p->lock);
    for (;;) {
        while (!p->quit && p->round == seen) pthread_cond_wait(&p->wake, &p->lock);
        if (p->quit) break;
        seen = p->round;
        Reads *r = p->reads;
        pthread_mutex_unlock(&p->lock);
        read_jobs(r, p->stage[index]);
        pthread_mutex_lock(&p->lock);
        if (--p->running == 0) pthread_cond_signal(&p->done);
    }
    pthread_mutex_unlock(&p->lock);
    return NULL;
}

/* Starts readers until `want` of them (besides the acquiring thread) exist; fewer when a thread or a stage cannot be had. */
static void start_readers(QW4ExpertPool *p, uint32_t want) {
    const size_t widest = widest_matrix(p);
    while (p->started < want && p->started < QW4_POOL_MAX_READERS) {
        const uint32_t index = p->started;
        if (!p->stage[index] && pf_hip_stage_create(widest, &p->stage[index]) != PF_HIP_OK) break;
        ReaderArg *arg = malloc(sizeof *arg);
        if (!arg) break;
        arg->p = p; arg->index = index; arg->round = p->round;   /* (only the acquiring thread changes it, and it is here) */
        if (pthread_create(&p->thread[index], NULL, reader_main, arg)) { free(arg); break; }
        p->started++;
    }
}

/* The misses of an acquire, read together: the pool's readers and this thread.  0, or -1 if a read or a store failed. */
static int read_misses(QW4ExpertPool *p, uint32_t layer, uint32_t misses) {
    Reads reads = {.p = p, .layer = layer, .misses = misses};
    atomic_init(&reads.next, 0);
    atomic_init(&reads.failed, 0);
    uint32_t width = p->readers < misses * 3 ? p->readers : misses * 3;
    if (width > QW4_POOL_MAX_READERS) width = QW4_POOL_MAX_READERS;
    PfHipStage **mine = &p->stage[QW4_POOL_MAX_READERS];
    if (!*mine && pf_hip_stage_create(widest_matrix(p), mine) != PF_HIP_OK) return -1;
    if (width > 1) start_readers(p, width - 1);
    pthread_mutex_lock(&p->lock);
    p->reads = &reads;
    p->running = p->started;      /* every started reader wakes, also those this acquire has no job for */
    p->round++;
    pthread_cond_broadcast(&p->wake);
    pthread_mutex_unlock(&p->lock);
    read_jobs(&reads, *mine);     /* this thread reads too; alone when no other could be started */
    pthread_mutex_lock(&p->lock);
    while (p->running) pthread_cond_wait(&p->done, &p->lock);
    p->reads = NULL;
    pthread_mutex_unlock(&p->lock);
    return atomic_load(&reads.failed) ? -1 : 0;
}

static uint64_t now_ns(void) {
    struct timespec t;
    clock_gettime(CLOCK_MONOTONIC, &t);
    return (uint64_t)t.tv_sec * 1000000000ull + (uint64_t)t.tv_nsec;
}

int qw4_pool_acquire(QW4ExpertPool *p, uint32_t layer, const uint32_t *experts, size_t n, uint32_t *slots) {
    if (!p || layer >= p->n_layers || (n && (!experts || !slots))) return -1;
    const uint64_t t0 = now_ns();
    p->used = true;
    uint32_t misses = 0;
    int rc = 0;
    /* pass 1: slots and victims, in list order */
    for (size_t i = 0; i < n && !rc; i++) {
        if (experts[i] >= p->experts) { qw4_pool_release(p, slots, i); rc = -1; break; }
        const uint32_t key = layer * p->experts + experts[i];
        uint32_t s = p->where[key];
        if (s != NO_SLOT) {
            p->stats.hits++;
        } else {
            for (uint32_t c = 0; c < p->slots; c++)   /* oldest stamp among the unpinned */
                if (!p->pins[c] && (s == NO_SLOT || p->stamp[c] < p->stamp[s])) s = c;
            if (s == NO_SLOT) { qw4_pool_release(p, slots, i); rc = -1; break; }
            if (p->holds[s] != NO_SLOT) { p->where[p->holds[s]] = NO_SLOT; p->stats.evictions++; }
            p->holds[s] = key;
            p->where[key] = s;
            p->stats.misses++;
            p->stats.bytes_read += p->bytes[0] + p->bytes[1] + p->bytes[2];
            p->new_slot[misses] = s;
            p->new_expert[misses] = experts[i];
            misses++;
        }
        p->pins[s]++;
        p->stamp[s] = p->clock++;
        slots[i] = s;
    }
    /* pass 2: the misses, read together */
    if (!rc && misses && read_misses(p, layer, misses)) { qw4_pool_release(p, slots, n); rc = -1; }
    if (rc)   /* the slots this call took hold nothing usable: forget them (their recency stays) */
        for (uint32_t j = 0; j < misses; j++) {
            p->where[p->holds[p->new_slot[j]]] = NO_SLOT;
            p->holds[p->new_slot[j]] = NO_SLOT;
        }
    p->stats.acquire_ns += now_ns() - t0;
    return rc;
}
