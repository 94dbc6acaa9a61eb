/*
 * sigref.c -- CPU oracle for the truncated path signature (TEST INFRASTRUCTURE ONLY).
 *
 * Plain-C restatement of the reference CPU algorithm (forward Horner sweep,
 * naive Chen sweep, reverse sweep with un-multiplication), threaded over
 * contiguous batch chunks the way the reference does it.  Used by the tests as
 * the checker and by the benchmark as the CPU baseline; the shipped GPU library
 * never links it.
 *
 * How each function is pinned independently of this file is listed in
 * tests/test_oracle.py: the reference's own golden vectors (iisignature values
 * for forward with both augmentations and for backward), the reference's
 * hand-computed known-answer tests, closed forms (straight line, d = 1, Chen,
 * time reversal, shuffle), a brute-force iterated-sum evaluation and central
 * finite differences.
 */
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>
#include "sigref.h"

/* siglib/cpsig/cp_utils.cpp:22-38 power(): 0 signals overflow */
static uint64_t pow_u64(uint64_t base, uint64_t e)
{
    uint64_t r = 1;
    while (e > 0) {
        if (e & 1) {
            if (r != 0 && base > UINT64_MAX / r) return 0;
            r *= base;
        }
        e >>= 1;
        if (e > 0) {
            if (base != 0 && base > UINT64_MAX / base) return 0;
            base *= base;
        }
    }
    return r;
}

uint64_t sigref_sig_length(uint64_t d, uint64_t degree)
{
    if (d == 0) return 1;
    if (d == 1) return degree + 1;
    const uint64_t p = pow_u64(d, degree + 1);
    return p ? (p - 1) / (d - 1) : 0;
}

int sigref_level_index(uint64_t *lvl, uint64_t d, uint64_t n)
{
    lvl[0] = 0;
    for (uint64_t i = 1; i < n; ++i) {
        if (d != 0 && lvl[i - 1] > UINT64_MAX / d) return 10;
        const uint64_t m = lvl[i - 1] * d;
        if (m > UINT64_MAX - 1) return 10;
        lvl[i] = m + 1;
    }
    return 0;
}

int sigref_max_threads(void)
{
    long n = sysconf(_SC_NPROCESSORS_ONLN);
    return n > 0 ? (int)n : 1;
}

typedef struct {
    void *ctx;
    void (*worker)(void *, uint64_t, uint64_t);
    uint64_t b0, b1;
} chunk_t;

static void *chunk_main(void *arg)
{
    chunk_t *c = (chunk_t *)arg;
    c->worker(c->ctx, c->b0, c->b1);
    return NULL;
}

void sigref_run_batch(uint64_t batch, int n_jobs, void *ctx, void (*worker)(void *, uint64_t, uint64_t))
{
    if (batch == 0) return;
    int max_threads = n_jobs > 0 ? n_jobs : sigref_max_threads() + 1 + n_jobs;
    if (max_threads < 1) max_threads = 1;
    /* siglib/cpsig/multithreading.h:47-60: serial when n_jobs == 1 or batch == 1 */
    if (max_threads == 1 || batch == 1) { worker(ctx, 0, batch); return; }
    const uint64_t nt = (uint64_t)max_threads < batch ? (uint64_t)max_threads : batch;
    const uint64_t q = batch / nt, r = batch % nt;
    pthread_t *th = (pthread_t *)malloc(nt * sizeof(pthread_t));
    chunk_t *ch = (chunk_t *)malloc(nt * sizeof(chunk_t));
    for (uint64_t t = 0; t < nt; ++t) {
        ch[t].ctx = ctx; ch[t].worker = worker;
        ch[t].b0 = t * q + (t < r ? t : r);
        ch[t].b1 = ch[t].b0 + q + (t < r ? 1 : 0);
        if (pthread_create(&th[t], NULL, chunk_main, &ch[t]) != 0) {
            chunk_main(&ch[t]);
            th[t] = 0;
        }
    }
    for (uint64_t t = 0; t < nt; ++t)
        if (th[t]) pthread_join(th[t], NULL);
    free(th); free(ch);
}

#define REAL float
#define SUF _f
#include "sigref_impl.h"
#undef REAL
#undef SUF

#define REAL double
#define SUF _d
#include "sigref_impl.h"
#undef REAL
#undef SUF
