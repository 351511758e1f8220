/* cpu_bench.c - TEST / BENCH INFRASTRUCTURE: times the CPU expert path of one routed decode layer on this host's cores.
 *
 * Used only by bench.py's cpu_baseline leg.  The method is the reference's own CPU bench (src/core/glm_cpu_bench.cpp:1-30):
 * a persistent spinning pool of pinned threads (one per physical core, include/strata/kernels/cpu/pool.hpp:66-72), expert
 * sets larger than the last-level cache rotating so every call streams its weights from DRAM, rounds of calls, the median.
 * A layer call is what ExpertPool::run_split_multi_native does (include/strata/kernels/cpu/pool.hpp:120-131): every routed
 * expert split by rows across all threads - gate/up rows, then the intermediate's quantization, then the down rows - and
 * the weighted sum in slot order (src/kernels/cuda/native_moe.cu:36-52).
 *
 * The row kernels are passed in: the reference's own iq256_gu_rows / iq256_rows (src/kernels/cpu/iq_avx2.cpp, through
 * oracle/_ref) where that build travelled, else this directory's plain-C restatement.
 */
#define _GNU_SOURCE
#include <pthread.h>
#include <sched.h>
#include <stdatomic.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "maya_oracle.h"

typedef void (*mo_gu_fn)(int type, const uint8_t* blob, size_t gu_row, size_t up_off, int n, const void* const* act, int nt,
                         float* const* ff, int r0, int r1);
typedef void (*mo_rows_fn)(int type, const uint8_t* w, size_t row_bytes, int n, const void* const* act, int nt,
                           float* const* out, int r0, int r1);

static void port_gu(int type, const uint8_t* blob, size_t gu_row, size_t up_off, int n, const void* const* act, int nt,
                    float* const* ff, int r0, int r1) {
    mo_gu_rows(type, blob, blob + up_off, gu_row, n, act, nt, ff, r0, r1, __builtin_inff());
}
static void port_rows(int type, const uint8_t* w, size_t row_bytes, int n, const void* const* act, int nt, float* const* out,
                      int r0, int r1) {
    mo_rows(type, w, row_bytes, n, act, nt, out, r0, r1);
}

#define MAXK 16

typedef struct {
    int type, k, n_embd, n_ff, n_threads, n_sets, rounds;
    double max_seconds;
    const uint8_t* const* blobs; /* [n_sets * k] */
    const float* weights;        /* [n_sets * k] */
    const float* x;
    mo_gu_fn gu;
    mo_rows_fn rows;
    size_t gu_row, d_row, up_off, down_off;
    uint8_t* xq;       /* Q8_K of x */
    float* h;          /* [k][n_ff] */
    uint8_t* hq;       /* [k] Q8_K rows of h */
    size_t hq_stride;
    float* part;       /* [k][n_embd] */
    float* out;        /* [n_embd] */
    double* times;
    int n_done;
    const int* cpus;
    atomic_int arrived;
    atomic_int phase;
    atomic_int stop;
} bench_t;

typedef struct {
    bench_t* b;
    int tid;
} worker_t;

static double now_s(void) {
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double) ts.tv_sec + 1e-9 * (double) ts.tv_nsec;
}

/* a sense-reversing spin barrier over the pool's threads (the reference's pool spins too: no futex on the token path) */
static void barrier(bench_t* b, int* sense) {
    *sense ^= 1;
    if (atomic_fetch_add(&b->arrived, 1) == b->n_threads - 1) {
        atomic_store(&b->arrived, 0);
        atomic_store(&b->phase, *sense);
    } else {
        while (atomic_load(&b->phase) != *sense) __builtin_ia32_pause();
    }
}

static void layer_call(bench_t* b, int tid, int set, int* sense) {
    const int T = b->n_threads, k = b->k;
    const uint8_t* const* blobs = b->blobs + (size_t) set * k;
    if (tid == 0) mo_quant_act(b->type, b->x, b->n_embd, b->xq);
    barrier(b, sense);
    const void* act[1] = {b->xq};
    {
        const int r0 = (int) ((int64_t) b->n_ff * tid / T), r1 = (int) ((int64_t) b->n_ff * (tid + 1) / T);
        for (int e = 0; e < k; ++e) {
            float* ff[1] = {b->h + (size_t) e * b->n_ff};
            if (r1 > r0) b->gu(b->type, blobs[e], b->gu_row, b->up_off, b->n_embd, act, 1, ff, r0, r1);
        }
    }
    barrier(b, sense);
    for (int e = tid; e < k; e += T) mo_quant_act(b->type, b->h + (size_t) e * b->n_ff, b->n_ff, b->hq + (size_t) e * b->hq_stride);
    barrier(b, sense);
    {
        const int r0 = (int) ((int64_t) b->n_embd * tid / T), r1 = (int) ((int64_t) b->n_embd * (tid + 1) / T);
        for (int e = 0; e < k; ++e) {
            const void* ha[1] = {b->hq + (size_t) e * b->hq_stride};
            float* o[1] = {b->part + (size_t) e * b->n_embd};
            if (r1 > r0) b->rows(b->type, blobs[e] + b->down_off, b->d_row, b->n_ff, ha, 1, o, r0, r1);
        }
        /* the weighted sum of this thread's own columns, slot order, each step rounded (no barrier needed: own rows) */
        const float* w = b->weights + (size_t) set * k;
        for (int c = r0; c < r1; ++c) {
            float s = w[0] * b->part[c];
            for (int e = 1; e < k; ++e) s = s + w[e] * b->part[(size_t) e * b->n_embd + c];
            b->out[c] = s;
        }
    }
    barrier(b, sense);
}

static void* worker(void* arg) {
    worker_t* w = (worker_t*) arg;
    bench_t* b = w->b;
    if (b->cpus) {
        cpu_set_t set;
        CPU_ZERO(&set);
        CPU_SET(b->cpus[w->tid], &set);
        pthread_setaffinity_np(pthread_self(), sizeof set, &set); /* refused: the thread stays where the scheduler puts it */
    }
    int sense = 0;
    /* warm-up: one pass over the sets (page the weights in, settle the clocks) */
    for (int s = 0; s < b->n_sets; ++s) layer_call(b, w->tid, s, &sense);
    const double t_begin = now_s();
    int call = 0;
    for (int r = 0; r < b->rounds; ++r) {
        for (int s = 0; s < b->n_sets; ++s) {
            const double t0 = now_s();
            layer_call(b, w->tid, s, &sense);
            if (w->tid == 0) b->times[call] = now_s() - t0;
            ++call;
        }
        /* thread 0 decides whether the time is up; every thread reads the same decision after the barrier */
        if (w->tid == 0 && r >= 6 && now_s() - t_begin > b->max_seconds) atomic_store(&b->stop, 1);
        barrier(b, &sense);
        if (atomic_load(&b->stop)) break;
    }
    if (w->tid == 0) b->n_done = call;
    return NULL;
}

/* Times `rounds` passes (at least 7, then until max_seconds) over n_sets sets of k routed experts of one type; a call is
 * one layer on one token.  times[rounds * n_sets] receives each call's seconds, *n_done their count; out0[n_embd] the
 * output of the LAST call (set (n_done - 1) % n_sets).  gu / rows NULL: the plain-C restatement.  cpus: the logical CPU to
 * pin each thread to, or NULL.  Returns 0, or 1 on a bad argument / failed allocation. */
int mo_bench_layer(int type, const uint8_t* const* blobs, int n_sets, int k, int n_embd, int n_ff, const float* x,
                   const float* weights, mo_gu_fn gu, mo_rows_fn rows, int n_threads, const int* cpus, int rounds,
                   double max_seconds, double* times, int* n_done, float* out_last) {
    if (k < 1 || k > MAXK || n_sets < 1 || n_threads < 1 || n_threads > 256 || rounds < 1 || mo_block_values(type) != 256) return 1;
    bench_t b;
    memset(&b, 0, sizeof b);
    b.type = type, b.k = k, b.n_embd = n_embd, b.n_ff = n_ff, b.n_threads = n_threads, b.n_sets = n_sets, b.rounds = rounds;
    b.max_seconds = max_seconds;
    b.blobs = blobs, b.weights = weights, b.x = x;
    b.gu = gu ? gu : port_gu;
    b.rows = rows ? rows : port_rows;
    b.gu_row = mo_row_bytes(type, n_embd);
    b.d_row = mo_row_bytes(type, n_ff);
    b.up_off = b.gu_row * (size_t) n_ff;
    b.down_off = 2 * b.up_off;
    b.hq_stride = (mo_act_bytes(type, n_ff) + 63) & ~(size_t) 63;
    b.xq = (uint8_t*) aligned_alloc(64, (mo_act_bytes(type, n_embd) + 63) & ~(size_t) 63);
    b.h = (float*) aligned_alloc(64, sizeof(float) * (size_t) k * n_ff);
    b.hq = (uint8_t*) aligned_alloc(64, b.hq_stride * (size_t) k);
    b.part = (float*) aligned_alloc(64, sizeof(float) * (size_t) k * n_embd);
    b.out = out_last;
    b.times = times;
    b.cpus = cpus;
    if (!b.xq || !b.h || !b.hq || !b.part) return 1;
    pthread_t th[256];
    worker_t wk[256];
    for (int t = 0; t < n_threads; ++t) {
        wk[t].b = &b;
        wk[t].tid = t;
        if (pthread_create(&th[t], NULL, worker, &wk[t]) != 0) {
            if (t == 0) return 1;
            abort(); /* the threads already started wait for the whole pool at their first barrier */
        }
    }
    for (int t = 0; t < n_threads; ++t) pthread_join(th[t], NULL);
    *n_done = b.n_done;
    free(b.xq), free(b.h), free(b.hq), free(b.part);
    return 0;
}
