/* CPU baseline harness (test infrastructure, like the rest of this directory).
 *
 * Times the oracle's kernels on the host with the reference's CPU discipline, so that a GPU
 * figure can be printed beside "the same seeded workload on this machine's cores":
 *
 *   - a persistent pool of workers parked on a condition variable, worker i pinned to CPU i,
 *     run(n, body) = dispatch to workers 0..n-1 and wait for all of them
 *     (reference: src/cpu/thread_pool.cpp:23-102, src/cpu/cpu_peak.h:75-102);
 *   - run_workload: warm-up dispatches, a settle phase before multi-threaded runs so the package
 *     is in the clock state of that thread count, an adaptive probe that grows the batch until a
 *     dispatch lasts 2 ms, pick_iters towards the time budget (cap 1e8), ONE timed dispatch whose
 *     body loops `iters` times itself (reference: src/cpu/cpu_peak.cpp:46-128,
 *     src/common/common.cpp:35-45);
 *   - measure: the body at 1 thread ("ST") and at every logical core ("MT"), value =
 *     units_per_iter * threads / (us * 1e3) in giga-units (reference:
 *     src/cpu/compute_common.h:21-60).
 *
 * Only tests and the cpu_baseline leg of the benchmark driver load this.  The built-in bodies call
 * the oracle's own functions (no fast-math, no contraction), so what is timed is the checker; the
 * *_fn entry points time kernels handed in as function pointers instead, which is how the
 * reference's own CPU kernels are timed where a build of them exists.
 */
#define _GNU_SOURCE
#include <math.h>
#include <omp.h>
#include <pthread.h>
#include <sched.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>
#include <unistd.h>

/* oracle.c */
void orc_fill_f32(float *dst, uint64_t n, uint64_t seed, uint32_t stream, int dist, uint64_t first);
void orc_global_bandwidth_range(int width, const float *in, uint64_t n_floats, uint64_t T, uint64_t t0, uint64_t t1,
                                float *out);
int orc_compute_mad(int kind, int width, uint64_t seed, uint64_t first, uint64_t n, uint32_t steps, void *out);
int orc_mfma_dense(int kind, const void *A, const void *B, const uint8_t *scaleA, const uint8_t *scaleB, void *out,
                   double *abs_out, uint32_t waves, uint32_t iters);
int orc_gemm_tile(int fmt, const void *A, const void *B, uint32_t K, uint32_t lda, uint32_t ldb, uint32_t m0,
                  uint32_t n0, uint32_t tm, uint32_t tn, double scale, double *C);
void orc_fill_normal_codes(int fmt, double sigma, uint64_t seed, uint32_t stream, uint64_t first, uint64_t n, void *out);
void orc_fill_int8(uint64_t seed, uint32_t stream, uint64_t first, uint64_t n, int8_t *out);
void orc_fill_bf16(uint16_t *dst, uint64_t n, uint64_t seed, uint32_t stream, int dist, uint64_t first);

typedef void (*cpuh_body)(void *ctx, int tid, uint64_t iters);

/* ------------------------------------------------------------------------- */
/* Thread pool                                                                 */
/* ------------------------------------------------------------------------- */
typedef struct cpuh_pool {
    int n_max;
    pthread_t *threads;
    pthread_mutex_t mtx;
    pthread_cond_t cv_start, cv_done;
    uint64_t generation;
    int stop, active, remaining;
    cpuh_body job;
    void *job_ctx;
    uint64_t job_iters;
    int *pinned_cpu;   /* what each worker is pinned to, -1 if pinning was refused */
} cpuh_pool;

typedef struct { cpuh_pool *pool; int tid; } worker_arg;

static void *worker_loop(void *argp)
{
    worker_arg *arg = (worker_arg *)argp;
    cpuh_pool *p = arg->pool;
    const int tid = arg->tid;
    free(arg);

    cpu_set_t set;
    CPU_ZERO(&set);
    CPU_SET(tid, &set);
    p->pinned_cpu[tid] = sched_setaffinity(0, sizeof(set), &set) == 0 ? tid : -1;
    omp_set_num_threads(1);   /* oracle functions carry OpenMP loops: inside a worker they stay on this thread */

    uint64_t my_gen = 0;
    for (;;) {
        cpuh_body job = NULL;
        void *ctx = NULL;
        uint64_t iters = 0;
        pthread_mutex_lock(&p->mtx);
        while (!p->stop && p->generation == my_gen) pthread_cond_wait(&p->cv_start, &p->mtx);
        if (p->stop) { pthread_mutex_unlock(&p->mtx); return NULL; }
        my_gen = p->generation;
        if (tid < p->active) { job = p->job; ctx = p->job_ctx; iters = p->job_iters; }
        pthread_mutex_unlock(&p->mtx);
        if (job) {
            job(ctx, tid, iters);
            pthread_mutex_lock(&p->mtx);
            if (--p->remaining == 0) pthread_cond_signal(&p->cv_done);
            pthread_mutex_unlock(&p->mtx);
        }
    }
}

cpuh_pool *cpuh_pool_create(int max_threads)
{
    if (max_threads < 1) max_threads = 1;
    cpuh_pool *p = (cpuh_pool *)calloc(1, sizeof(*p));
    if (!p) return NULL;
    p->n_max = max_threads;
    p->threads = (pthread_t *)calloc((size_t)max_threads, sizeof(pthread_t));
    p->pinned_cpu = (int *)calloc((size_t)max_threads, sizeof(int));
    pthread_mutex_init(&p->mtx, NULL);
    pthread_cond_init(&p->cv_start, NULL);
    pthread_cond_init(&p->cv_done, NULL);
    for (int t = 0; t < max_threads; t++) {
        worker_arg *a = (worker_arg *)malloc(sizeof(*a));
        a->pool = p;
        a->tid = t;
        p->pinned_cpu[t] = -2;
        pthread_create(&p->threads[t], NULL, worker_loop, a);
    }
    return p;
}

void cpuh_pool_destroy(cpuh_pool *p)
{
    if (!p) return;
    pthread_mutex_lock(&p->mtx);
    p->stop = 1;
    p->generation++;
    pthread_cond_broadcast(&p->cv_start);
    pthread_mutex_unlock(&p->mtx);
    for (int t = 0; t < p->n_max; t++) pthread_join(p->threads[t], NULL);
    pthread_mutex_destroy(&p->mtx);
    pthread_cond_destroy(&p->cv_start);
    pthread_cond_destroy(&p->cv_done);
    free(p->threads);
    free(p->pinned_cpu);
    free(p);
}

int cpuh_pool_max_threads(const cpuh_pool *p) { return p->n_max; }

/* CPU worker `tid` is pinned to, -1 if the OS refused, -2 if the worker has not started yet. */
int cpuh_pool_pinned_cpu(const cpuh_pool *p, int tid) { return tid >= 0 && tid < p->n_max ? p->pinned_cpu[tid] : -1; }

/* body(ctx, tid, iters) on workers 0..n-1; returns when all are done. */
void cpuh_pool_run(cpuh_pool *p, int n, cpuh_body body, void *ctx, uint64_t iters)
{
    if (n < 1) n = 1;
    if (n > p->n_max) n = p->n_max;
    pthread_mutex_lock(&p->mtx);
    p->job = body;
    p->job_ctx = ctx;
    p->job_iters = iters;
    p->active = n;
    p->remaining = n;
    p->generation++;
    pthread_cond_broadcast(&p->cv_start);
    while (p->remaining != 0) pthread_cond_wait(&p->cv_done, &p->mtx);
    p->job = NULL;
    pthread_mutex_unlock(&p->mtx);
}

/* ------------------------------------------------------------------------- */
/* Timing discipline                                                           */
/* ------------------------------------------------------------------------- */
unsigned cpuh_pick_iters(double per_iter_us, unsigned target_us, unsigned forced, unsigned max_iters)
{
    if (forced) return forced;
    if (target_us == 0) target_us = 5000000;
    if (per_iter_us < 1.0) per_iter_us = 1.0;
    double want = (double)target_us / per_iter_us;
    if (want < 1.0) want = 1.0;
    if (want > (double)max_iters) want = (double)max_iters;
    return (unsigned)want;
}

static double now_us(void)
{
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec * 1e6 + (double)ts.tv_nsec / 1e3;
}

/* Mean microseconds per iteration of `body` at n_threads; *iters_out = size of the timed batch. */
double cpuh_run_workload(cpuh_pool *p, int n_threads, cpuh_body body, void *ctx, unsigned warmup,
                         unsigned target_us, unsigned forced_iters, unsigned *iters_out)
{
    if (n_threads < 1) n_threads = 1;
    if (n_threads > p->n_max) n_threads = p->n_max;

    for (unsigned w = 0; w < warmup; w++) cpuh_pool_run(p, n_threads, body, ctx, 1);

    if (n_threads > 1) {
        /* a quarter of the budget, between 100 and 500 ms, at this thread count */
        double settle = (double)target_us / 4.0;
        if (settle < 100000.0) settle = 100000.0;
        if (settle > 500000.0) settle = 500000.0;
        const double w0 = now_us();
        uint64_t w_iters = 1;
        while (now_us() - w0 < settle) {
            cpuh_pool_run(p, n_threads, body, ctx, w_iters);
            if (w_iters < (1ull << 32)) w_iters *= 2;
        }
    }

    double per_iter_us = 1.0;
    if (!forced_iters) {
        uint64_t probe_iters = 1;
        double probe_us;
        for (;;) {
            const double p0 = now_us();
            cpuh_pool_run(p, n_threads, body, ctx, probe_iters);
            probe_us = now_us() - p0;
            if (probe_us >= 2000.0 || probe_iters >= (1ull << 24)) break;
            probe_iters *= 4;
        }
        per_iter_us = probe_us / (double)probe_iters;
        if (per_iter_us <= 0.0) per_iter_us = 0.01;
    }

    const unsigned iters = cpuh_pick_iters(per_iter_us, target_us, forced_iters, 100000000u);
    const double t0 = now_us();
    cpuh_pool_run(p, n_threads, body, ctx, iters);
    const double total = now_us() - t0;
    if (iters_out) *iters_out = iters;
    return total / (double)iters;
}

/* ------------------------------------------------------------------------- */
/* Workloads: the oracle's kernels as body(tid, iters)                         */
/* ------------------------------------------------------------------------- */
enum { CPUH_READ_FLOAT4 = 0, CPUH_MAD_F32 = 1, CPUH_MFMA_BF16 = 2, CPUH_MFMA_I8 = 3, CPUH_GEMM_BF16 = 4, CPUH_COUNT };

#define MAX_T 1024

typedef struct {
    int kind, n_threads;
    uint64_t seed;
    /* read */
    float *buf, *partials;
    uint64_t n_floats, T;
    /* mad */
    float *mad_out;
    /* mfma */
    void *A, *B;
    float *tiles;
    /* gemm */
    uint16_t *ga, *gb;
    double *gc;
    double sink[MAX_T];
} workload;

/* one iteration = this thread's contiguous share of the 2^20 partial sums, i.e. 1/n of the buffer */
static void body_read(void *c, int tid, uint64_t iters)
{
    workload *w = (workload *)c;
    const uint64_t t0 = w->T * (uint64_t)tid / (uint64_t)w->n_threads, t1 = w->T * (uint64_t)(tid + 1) / (uint64_t)w->n_threads;
    for (uint64_t i = 0; i < iters; i++) {
        orc_global_bandwidth_range(4, w->buf, w->n_floats, w->T, t0, t1, w->partials);
        w->sink[tid] += (double)w->partials[t0];
    }
}

/* one iteration = 8 work-items of the MAD chain (16 accumulators x 4096 dependent fma each);
 * successive iterations and threads take successive items of the 2^20 */
#define MAD_ITEMS 8
static void body_mad(void *c, int tid, uint64_t iters)
{
    workload *w = (workload *)c;
    float *out = w->mad_out + (size_t)tid * MAD_ITEMS;
    for (uint64_t i = 0; i < iters; i++) {
        const uint64_t first = (((uint64_t)tid << 14) + i) * MAD_ITEMS % (1ull << 20);
        orc_compute_mad(0, 4, w->seed, first, MAD_ITEMS, 4096, out);
        w->sink[tid] += (double)out[0];
    }
}

/* one iteration = one emulated matrix instruction on each of a wave's 4 chains */
static void body_mfma(void *c, int tid, uint64_t iters)
{
    workload *w = (workload *)c;
    float *out = w->tiles + (size_t)tid * 4 * 256;
    const int kind = w->kind == CPUH_MFMA_BF16 ? 1 : 4;   /* C ABI numbering: bf16 16x16x32, i8 16x16x64 */
    for (uint64_t i = 0; i < iters; i++) {
        orc_mfma_dense(kind, w->A, w->B, NULL, NULL, out, NULL, 1, 1);
        w->sink[tid] += (double)out[0];
    }
}

/* one iteration = one 64x64 tile of the 8192-deep bf16 GEMM */
#define GEMM_K 8192u
#define GEMM_T 64u
static void body_gemm(void *c, int tid, uint64_t iters)
{
    workload *w = (workload *)c;
    double *C = w->gc + (size_t)tid * GEMM_T * GEMM_T;
    for (uint64_t i = 0; i < iters; i++) {
        orc_gemm_tile(1, w->ga, w->gb, GEMM_K, GEMM_K, GEMM_K, 0, 0, GEMM_T, GEMM_T, 1.0, C);
        w->sink[tid] += C[0];
    }
}

typedef struct {
    double us_st, us_mt;           /* mean microseconds per iteration */
    unsigned iters_st, iters_mt;   /* size of the timed batch */
    int threads_mt;                /* workers of the MT run */
    int pinned;                    /* workers whose pinning the OS accepted */
    double units_per_iter_st;      /* flops / ops / bytes one iteration is worth at 1 thread, per thread */
    double units_per_iter_mt;      /* the same at threads_mt threads, per thread */
    double giga_st, giga_mt;       /* units * threads / (us * 1e3) */
} cpuh_result;

/* Runs workload `kind` at 1 thread and at every worker of the pool.  target_us is the time budget
 * of each of the two timed batches.  Returns 0, -1 for an unknown kind, -3 when out of memory. */
int cpuh_measure(cpuh_pool *p, int kind, uint64_t seed, unsigned warmup, unsigned target_us, cpuh_result *r)
{
    if (kind < 0 || kind >= CPUH_COUNT || !r) return -1;
    const int n = p->n_max > MAX_T ? MAX_T : p->n_max;
    workload *w = (workload *)calloc(1, sizeof(*w));
    if (!w) return -3;
    w->kind = kind;
    w->seed = seed;
    cpuh_body body = NULL;
    double units_st = 0.0, units_mt = 0.0;
    int rc = 0;
    switch (kind) {
    case CPUH_READ_FLOAT4:
        w->n_floats = 1ull << 26;
        w->T = 1ull << 20;
        w->buf = (float *)aligned_alloc(64, w->n_floats * sizeof(float));
        w->partials = (float *)aligned_alloc(64, w->T * sizeof(float));
        if (!w->buf || !w->partials) { rc = -3; break; }
        orc_fill_f32(w->buf, w->n_floats, seed, 0, 0, 0);
        body = body_read;
        units_st = (double)w->n_floats * 4.0;              /* the whole buffer per iteration */
        units_mt = (double)w->n_floats * 4.0 / (double)n;  /* each thread its share */
        break;
    case CPUH_MAD_F32:
        w->mad_out = (float *)calloc((size_t)n * MAD_ITEMS, sizeof(float));
        if (!w->mad_out) { rc = -3; break; }
        body = body_mad;
        units_st = units_mt = (double)MAD_ITEMS * 16.0 * 4096.0 * 2.0;
        break;
    case CPUH_MFMA_BF16:
    case CPUH_MFMA_I8: {
        const int K = kind == CPUH_MFMA_BF16 ? 32 : 64, eb = kind == CPUH_MFMA_BF16 ? 2 : 1;
        const size_t elems = (size_t)4 * 16 * (size_t)K;
        w->A = malloc(elems * (size_t)eb);
        w->B = malloc(elems * (size_t)eb);
        w->tiles = (float *)calloc((size_t)n * 4 * 256, sizeof(float));
        if (!w->A || !w->B || !w->tiles) { rc = -3; break; }
        if (kind == CPUH_MFMA_BF16) {
            orc_fill_normal_codes(1, 0.01, seed, 2, 0, elems, w->A);
            orc_fill_normal_codes(1, 0.01, seed, 3, 0, elems, w->B);
        } else {
            orc_fill_int8(seed, 2, 0, elems, (int8_t *)w->A);
            orc_fill_int8(seed, 3, 0, elems, (int8_t *)w->B);
        }
        body = body_mfma;
        units_st = units_mt = 4.0 * 2.0 * 16.0 * 16.0 * (double)K;
        break;
    }
    case CPUH_GEMM_BF16:
        w->ga = (uint16_t *)malloc((size_t)GEMM_T * GEMM_K * 2);
        w->gb = (uint16_t *)malloc((size_t)GEMM_T * GEMM_K * 2);
        w->gc = (double *)calloc((size_t)n * GEMM_T * GEMM_T, sizeof(double));
        if (!w->ga || !w->gb || !w->gc) { rc = -3; break; }
        orc_fill_bf16(w->ga, (uint64_t)GEMM_T * GEMM_K, seed, 7, 1, 0);
        orc_fill_bf16(w->gb, (uint64_t)GEMM_T * GEMM_K, seed, 8, 1, 0);
        body = body_gemm;
        units_st = units_mt = 2.0 * (double)GEMM_T * (double)GEMM_T * (double)GEMM_K;
        break;
    }
    if (rc == 0) {
        memset(r, 0, sizeof(*r));
        w->n_threads = 1;
        r->us_st = cpuh_run_workload(p, 1, body, w, warmup, target_us, 0, &r->iters_st);
        w->n_threads = n;
        r->us_mt = cpuh_run_workload(p, n, body, w, warmup, target_us, 0, &r->iters_mt);
        r->threads_mt = n;
        for (int t = 0; t < n; t++) r->pinned += p->pinned_cpu[t] == t;
        r->units_per_iter_st = units_st;
        r->units_per_iter_mt = units_mt;
        r->giga_st = r->us_st > 0.0 ? units_st / (r->us_st * 1e3) : -1.0;
        r->giga_mt = r->us_mt > 0.0 ? units_mt * (double)n / (r->us_mt * 1e3) : -1.0;
        volatile double keep = 0.0;
        for (int t = 0; t < n; t++) keep += w->sink[t];
        (void)keep;
    }
    free(w->buf); free(w->partials); free(w->mad_out); free(w->A); free(w->B); free(w->tiles);
    free(w->ga); free(w->gb); free(w->gc); free(w);
    return rc;
}

/* ------------------------------------------------------------------------- */
/* Kernels handed in as function pointers (the reference's own CPU kernels, where a build of them
 * exists): the chain signature and the streaming-read signature of src/cpu/cpu_kernels.h:62-66.   */
typedef double (*cpuh_chain_fn)(uint64_t outer);
typedef uint64_t (*cpuh_read_fn)(const float *p, size_t m, uint64_t iters);
typedef void (*cpuh_populate_fn)(float *p, unsigned long long n);

typedef struct {
    cpuh_chain_fn chain;
    cpuh_read_fn read;
    cpuh_populate_fn populate;
    float *buf;
    uint64_t n_floats;
    int n_threads;        /* threads of the dispatch being timed: the buffer is split among them */
    double sink[MAX_T];
    uint64_t xsink[MAX_T];
} fn_workload;

static void body_chain_fn(void *c, int tid, uint64_t iters)
{
    fn_workload *w = (fn_workload *)c;
    w->sink[tid] += w->chain(iters);
}

/* per-thread contiguous chunk, the last thread takes the remainder (src/cpu/bandwidth.cpp:283-288) */
static void chunk_of(const fn_workload *w, int tid, int n, uint64_t *lo, uint64_t *hi)
{
    const uint64_t per = w->n_floats / (uint64_t)n;
    *lo = (uint64_t)tid * per;
    *hi = tid == n - 1 ? w->n_floats : *lo + per;
}

static void body_read_fn(void *c, int tid, uint64_t iters)
{
    fn_workload *w = (fn_workload *)c;
    uint64_t lo, hi;
    chunk_of(w, tid, w->n_threads, &lo, &hi);
    w->xsink[tid] ^= w->read(w->buf + lo, (size_t)(hi - lo), iters);
}

static void body_first_touch(void *c, int tid, uint64_t iters)
{
    fn_workload *w = (fn_workload *)c;
    (void)iters;
    uint64_t lo, hi;
    chunk_of(w, tid, w->n_threads, &lo, &hi);
    w->populate(w->buf + lo, hi - lo);
}

static void finish(cpuh_pool *p, cpuh_result *r, int n, double units_st, double units_mt)
{
    r->threads_mt = n;
    r->pinned = 0;
    for (int t = 0; t < n; t++) r->pinned += p->pinned_cpu[t] == t;
    r->units_per_iter_st = units_st;
    r->units_per_iter_mt = units_mt;
    r->giga_st = r->us_st > 0.0 ? units_st / (r->us_st * 1e3) : -1.0;
    r->giga_mt = r->us_mt > 0.0 ? units_mt * (double)n / (r->us_mt * 1e3) : -1.0;
}

/* ------------------------------------------------------------------------- */
/* Any oracle kernel on operands the caller built: one descriptor, one body.                      */
/* The caller (the cpu_baseline leg of the benchmark driver) makes the seeded operands with the   */
/* same generator the GPU rows use and states what one iteration is worth.                         */
/* ------------------------------------------------------------------------- */
int orc_smfmac(int kind, const void *Ac, const uint8_t *meta, const void *B, void *out, double *abs_out, uint32_t waves,
               uint32_t iters);
int orc_gemm_tile2(int fmt_a, int fmt_b, const void *A, const void *B, uint32_t K, uint32_t lda, uint32_t ldb, uint32_t m0,
                   uint32_t n0, uint32_t tm, uint32_t tn, double scale, double *C);
int orc_gemm_mx_tile(const uint8_t *A, const uint8_t *B, const uint8_t *SA, const uint8_t *SB, uint32_t K, uint32_t m0,
                     uint32_t n0, uint32_t tm, uint32_t tn, double *C);

enum { CPUH_OP_MAD = 0, CPUH_OP_MFMA = 1, CPUH_OP_SMFMAC = 2, CPUH_OP_GEMM = 3, CPUH_OP_GEMM_MX = 4, CPUH_OP_READ = 5 };

typedef struct {
    int op;
    int kind;            /* MAD / MFMA / SMFMAC kind (C ABI numbering); GEMM: format of A */
    int width;           /* MAD: width or chains; READ: vector width; GEMM: format of B */
    uint64_t seed;       /* MAD */
    const void *p0, *p1, *p2, *p3;   /* MFMA: A, B, scaleA, scaleB; SMFMAC: Ac, meta, B; GEMM: A, B (MX: + SA, SB); READ: buffer */
    uint32_t K, tile;    /* GEMM: depth and tile edge */
    double scale;        /* GEMM */
    uint64_t n_floats, T;   /* READ: buffer length and number of partial sums */
} cpuh_op;

typedef struct {
    cpuh_op op;
    int n_threads;
    size_t out_stride;   /* bytes of result space per thread */
    uint8_t *out;
    double sink[MAX_T];
} op_workload;

#define OP_MAD_ITEMS 8
static void body_op(void *c, int tid, uint64_t iters)
{
    op_workload *w = (op_workload *)c;
    const cpuh_op *o = &w->op;
    void *out = w->out + (size_t)tid * w->out_stride;
    for (uint64_t i = 0; i < iters; i++) {
        switch (o->op) {
        case CPUH_OP_MAD: {
            const uint64_t first = (((uint64_t)tid << 14) + i) * OP_MAD_ITEMS % (1ull << 20);
            orc_compute_mad(o->kind, o->width, o->seed, first, OP_MAD_ITEMS, 4096, out);
            break;
        }
        case CPUH_OP_MFMA:
            orc_mfma_dense(o->kind, o->p0, o->p1, (const uint8_t *)o->p2, (const uint8_t *)o->p3, out, NULL, 1, 1);
            break;
        case CPUH_OP_SMFMAC:
            orc_smfmac(o->kind, o->p0, (const uint8_t *)o->p1, o->p2, out, NULL, 1, 1);
            break;
        case CPUH_OP_GEMM:
            orc_gemm_tile2(o->kind, o->width, o->p0, o->p1, o->K, o->K, o->K, 0, 0, o->tile, o->tile, o->scale, (double *)out);
            break;
        case CPUH_OP_GEMM_MX:
            orc_gemm_mx_tile((const uint8_t *)o->p0, (const uint8_t *)o->p1, (const uint8_t *)o->p2, (const uint8_t *)o->p3,
                             o->K, 0, 0, o->tile, o->tile, (double *)out);
            break;
        case CPUH_OP_READ: {
            /* this thread's contiguous share of the T partial sums; the partials are the shared result */
            const uint64_t t0 = o->T * (uint64_t)tid / (uint64_t)w->n_threads, t1 = o->T * (uint64_t)(tid + 1) / (uint64_t)w->n_threads;
            orc_global_bandwidth_range(o->width, (const float *)o->p0, o->n_floats, o->T, t0, t1, (float *)w->out);
            out = (float *)w->out + t0;
            break;
        }
        default:
            return;
        }
        w->sink[tid] += (double)*(const uint32_t *)out;
    }
}

/* Times the operation at 1 thread and at every worker.  units_st / units_mt: what one iteration of one thread
 * is worth (flop, op or byte) in the two runs (they differ only where the threads split one pass: READ). */
int cpuh_measure_op(cpuh_pool *p, const cpuh_op *op, double units_st, double units_mt, unsigned warmup, unsigned target_us,
                    cpuh_result *r)
{
    if (!op || !r || op->op < CPUH_OP_MAD || op->op > CPUH_OP_READ) return -1;
    const int n = p->n_max > MAX_T ? MAX_T : p->n_max;
    op_workload *w = (op_workload *)calloc(1, sizeof(*w));
    if (!w) return -3;
    w->op = *op;
    size_t total;
    if (op->op == CPUH_OP_READ) {
        w->out_stride = 0;
        total = (size_t)op->T * sizeof(float);
    } else {
        w->out_stride = op->op == CPUH_OP_GEMM || op->op == CPUH_OP_GEMM_MX ? (size_t)op->tile * op->tile * sizeof(double)
                        : op->op == CPUH_OP_MAD ? OP_MAD_ITEMS * 8 : 4 * 32 * 32 * sizeof(float);
        total = w->out_stride * (size_t)n;
    }
    w->out = (uint8_t *)aligned_alloc(64, (total + 63) / 64 * 64);
    if (!w->out) { free(w); return -3; }
    memset(w->out, 0, total);
    memset(r, 0, sizeof(*r));
    w->n_threads = 1;
    r->us_st = cpuh_run_workload(p, 1, body_op, w, warmup, target_us, 0, &r->iters_st);
    w->n_threads = n;
    r->us_mt = cpuh_run_workload(p, n, body_op, w, warmup, target_us, 0, &r->iters_mt);
    finish(p, r, n, units_st, units_mt);
    volatile double keep = 0.0;
    for (int t = 0; t < n; t++) keep += w->sink[t];
    (void)keep;
    free(w->out);
    free(w);
    return 0;
}

/* A compute chain at 1 thread and at every worker: value = ops_per_iter * threads / (us * 1e3). */
int cpuh_measure_chain_fn(cpuh_pool *p, cpuh_chain_fn fn, double ops_per_iter, unsigned warmup, unsigned target_us,
                          cpuh_result *r)
{
    if (!fn || !r) return -1;
    const int n = p->n_max > MAX_T ? MAX_T : p->n_max;
    fn_workload *w = (fn_workload *)calloc(1, sizeof(*w));
    if (!w) return -3;
    w->chain = fn;
    memset(r, 0, sizeof(*r));
    r->us_st = cpuh_run_workload(p, 1, body_chain_fn, w, warmup, target_us, 0, &r->iters_st);
    r->us_mt = cpuh_run_workload(p, n, body_chain_fn, w, warmup, target_us, 0, &r->iters_mt);
    finish(p, r, n, ops_per_iter, ops_per_iter);
    volatile double keep = 0.0;
    for (int t = 0; t < n; t++) keep += w->sink[t];
    (void)keep;
    free(w);
    return 0;
}

/* A streaming read over one shared array of n_floats, first-touched in parallel by the threads that
 * will read it and split into per-thread contiguous chunks; one iteration = one pass over the whole
 * array, value = n_floats * 4 / (us * 1e3) GB/s (src/cpu/bandwidth.cpp:274-321). */
int cpuh_measure_read_fn(cpuh_pool *p, cpuh_read_fn fn, cpuh_populate_fn populate, uint64_t n_floats, unsigned warmup,
                         unsigned target_us, cpuh_result *r)
{
    if (!fn || !populate || !r || n_floats == 0) return -1;
    const int n = p->n_max > MAX_T ? MAX_T : p->n_max;
    fn_workload *w = (fn_workload *)calloc(1, sizeof(*w));
    if (!w) return -3;
    w->read = fn;
    w->populate = populate;
    w->n_floats = n_floats / (uint64_t)n * (uint64_t)n;
    w->buf = (float *)aligned_alloc(64, w->n_floats * sizeof(float));
    if (!w->buf) { free(w); return -3; }
    w->n_threads = n;
    cpuh_pool_run(p, n, body_first_touch, w, 1);
    memset(r, 0, sizeof(*r));
    w->n_threads = 1;
    r->us_st = cpuh_run_workload(p, 1, body_read_fn, w, warmup, target_us, 0, &r->iters_st);
    w->n_threads = n;
    r->us_mt = cpuh_run_workload(p, n, body_read_fn, w, warmup, target_us, 0, &r->iters_mt);
    finish(p, r, n, (double)w->n_floats * 4.0, (double)w->n_floats * 4.0 / (double)n);
    volatile uint64_t keep = 0;
    for (int t = 0; t < n; t++) keep ^= w->xsink[t];
    (void)keep;
    free(w->buf);
    free(w);
    return 0;
}

/* The reference's buffer fill, restated (src/common/common.cpp:76-95): xorshift32 from 0xDEADBEEF per
 * call, bits forced to a finite positive float.  Every chunk a thread fills starts the sequence again. */
void cpuh_populate(float *p, unsigned long long n)
{
    uint32_t state = 0xDEADBEEFu;
    for (unsigned long long i = 0; i < n; i++) {
        state ^= state << 13;
        state ^= state >> 17;
        state ^= state << 5;
        const uint32_t bits = (state & 0x7F7FFFFFu) | 0x00800000u;
        memcpy(&p[i], &bits, sizeof(float));
    }
}

/* The other two rows of the reference's DRAM test (src/cpu/bandwidth.cpp:323-352): three arrays of
 * n_floats, first-touched in parallel, every thread working on its own contiguous chunk.
 *   copy  (kind 0): memcpy(A + lo, C + lo, chunk), 2 * n_floats * 4 bytes per iteration;
 *   triad (kind 1): A[i] = B[i] + 1.5f * C[i],      3 * n_floats * 4 bytes per iteration.
 * Timed at every worker only, as the reference does (ST fields of the result stay 0 / -1). */
typedef struct {
    float *a, *b, *c;
    uint64_t n_floats;
    int n_threads, kind;
    cpuh_populate_fn populate;
} stream_workload;

static void stream_chunk(const stream_workload *w, int tid, uint64_t *lo, uint64_t *hi)
{
    const uint64_t per = w->n_floats / (uint64_t)w->n_threads;
    *lo = (uint64_t)tid * per;
    *hi = tid == w->n_threads - 1 ? w->n_floats : *lo + per;
}

static void body_stream_touch(void *c, int tid, uint64_t iters)
{
    stream_workload *w = (stream_workload *)c;
    (void)iters;
    uint64_t lo, hi;
    stream_chunk(w, tid, &lo, &hi);
    w->populate(w->a + lo, hi - lo);
    w->populate(w->b + lo, hi - lo);
    w->populate(w->c + lo, hi - lo);
}

static void body_stream(void *c, int tid, uint64_t iters)
{
    stream_workload *w = (stream_workload *)c;
    uint64_t lo, hi;
    stream_chunk(w, tid, &lo, &hi);
    if (w->kind == 0) {
        for (uint64_t it = 0; it < iters; it++) {
            memcpy(w->a + lo, w->c + lo, (size_t)(hi - lo) * sizeof(float));
            __asm__ volatile("" ::: "memory");   /* every pass is done */
        }
    } else {
        const float s = 1.5f;
        float *restrict a = w->a;
        const float *restrict b = w->b, *restrict cc = w->c;
        for (uint64_t it = 0; it < iters; it++) {
            for (uint64_t i = lo; i < hi; i++) a[i] = b[i] + s * cc[i];
            __asm__ volatile("" ::: "memory");
        }
    }
}

int cpuh_measure_stream(cpuh_pool *p, cpuh_populate_fn populate, uint64_t n_floats, int kind, unsigned warmup,
                        unsigned target_us, cpuh_result *r, float *probe_out)
{
    if (!populate || !r || n_floats == 0 || (kind != 0 && kind != 1)) return -1;
    const int n = p->n_max > MAX_T ? MAX_T : p->n_max;
    stream_workload w;
    memset(&w, 0, sizeof(w));
    w.n_floats = n_floats;
    w.n_threads = n;
    w.kind = kind;
    w.populate = populate;
    w.a = (float *)aligned_alloc(64, (n_floats * sizeof(float) + 63) / 64 * 64);
    w.b = (float *)aligned_alloc(64, (n_floats * sizeof(float) + 63) / 64 * 64);
    w.c = (float *)aligned_alloc(64, (n_floats * sizeof(float) + 63) / 64 * 64);
    if (!w.a || !w.b || !w.c) { free(w.a); free(w.b); free(w.c); return -3; }
    cpuh_pool_run(p, n, body_stream_touch, &w, 1);
    memset(r, 0, sizeof(*r));
    r->us_mt = cpuh_run_workload(p, n, body_stream, &w, warmup, target_us, 0, &r->iters_mt);
    const double bytes = (kind == 0 ? 2.0 : 3.0) * (double)n_floats * 4.0;
    finish(p, r, n, bytes, bytes / (double)n);
    /* a few results, so that a test can check what the pass computed */
    if (probe_out) { probe_out[0] = w.a[0]; probe_out[1] = w.a[n_floats / 2]; probe_out[2] = w.a[n_floats - 1];
                     probe_out[3] = w.b[n_floats / 2]; probe_out[4] = w.c[n_floats / 2]; }
    free(w.a); free(w.b); free(w.c);
    return 0;
}

/* Test hook: a body that sleeps `ctx` microseconds per iteration, so the discipline can be checked
 * against a known per-iteration time. */
static void body_sleep(void *c, int tid, uint64_t iters)
{
    (void)tid;
    const unsigned us = *(const unsigned *)c;
    for (uint64_t i = 0; i < iters; i++) usleep(us);
}

double cpuh_time_sleep_body(cpuh_pool *p, int n_threads, unsigned sleep_us, unsigned target_us, unsigned *iters_out)
{
    return cpuh_run_workload(p, n_threads, body_sleep, &sleep_us, 2, target_us, 0, iters_out);
}

/* Test hook: every worker 0..n-1 adds (tid+1)*iters to slot tid of `counts`. */
static void body_count(void *c, int tid, uint64_t iters) { ((uint64_t *)c)[tid] += (uint64_t)(tid + 1) * iters; }

void cpuh_pool_count(cpuh_pool *p, int n, uint64_t iters, uint64_t *counts) { cpuh_pool_run(p, n, body_count, counts, iters); }
