/*
 * pool_harness.c -- host-only stand-in for the device allocator behind
 * xccl_amd/csrc/mc_pool.c, so that the freed-block cache can be tested
 * without a GPU.  Built by tests/test_mem_pool.py together with mc_pool.c.
 */
#include "mc_pool.h"

#include <pthread.h>
#include <stdatomic.h>
#include <stdlib.h>
#include <string.h>

static atomic_long n_alloc, n_free;
static atomic_int  fail_next; /* this many backing allocations fail */

static int backing_alloc(void **ptr, size_t len)
{
    if (atomic_load(&fail_next) > 0) {
        atomic_fetch_sub(&fail_next, 1);
        *ptr = NULL;
        return 2; /* "out of memory" */
    }
    *ptr = malloc(len ? len : 1);
    atomic_fetch_add(&n_alloc, 1);
    return *ptr ? 0 : 2;
}

static int backing_free(void *ptr)
{
    free(ptr);
    atomic_fetch_add(&n_free, 1);
    return 0;
}

void harness_configure(size_t limit)
{
    mc_pool_configure(backing_alloc, backing_free, limit);
}

long harness_backing_allocs(void) { return atomic_load(&n_alloc); }
long harness_backing_frees(void) { return atomic_load(&n_free); }
void harness_fail_next(int n) { atomic_store(&fail_next, n); }

/* One thread of the stress test: random allocations from a few size classes,
 * each block stamped with a value only this thread and slot use; a block
 * handed to two owners at once shows up as a corrupted stamp. */
typedef struct {
    int      id, iters;
    unsigned seed;
    long     errors;
} stress_arg_t;

static void *stress_thread(void *p)
{
    stress_arg_t *a = (stress_arg_t *)p;
    enum { HOLD = 8 };
    void    *held[HOLD]  = {0};
    size_t   bytes[HOLD] = {0};
    unsigned x           = a->seed;
    int      i, k;

    for (i = 0; i < a->iters; i++) {
        x = x * 1664525u + 1013904223u;
        k = (x >> 8) % HOLD;
        if (held[k] != NULL) {
            const unsigned char want = (unsigned char)(a->id * 16 + k);
            size_t              j;
            for (j = 0; j < bytes[k]; j += 509) {
                a->errors += ((unsigned char *)held[k])[j] != want;
            }
            a->errors += mc_pool_free(held[k]) != 0;
            held[k] = NULL;
        } else {
            bytes[k] = (size_t)4096 << ((x >> 16) % 6);
            bytes[k] += (x >> 24) % 3 * 1000;
            if (mc_pool_alloc((x >> 28) & 1, &held[k], bytes[k]) != 0) {
                a->errors++;
                held[k] = NULL;
                continue;
            }
            memset(held[k], a->id * 16 + k, bytes[k]);
        }
    }
    for (k = 0; k < HOLD; k++) {
        if (held[k] != NULL) {
            a->errors += mc_pool_free(held[k]) != 0;
        }
    }
    return NULL;
}

long harness_stress(int threads, int iters)
{
    pthread_t    th[16];
    stress_arg_t arg[16];
    long         errors = 0;
    int          t;

    if (threads > 16) {
        threads = 16;
    }
    for (t = 0; t < threads; t++) {
        arg[t] = (stress_arg_t){.id = t + 1, .iters = iters, .seed = 12345u + 77u * (unsigned)t, .errors = 0};
        pthread_create(&th[t], NULL, stress_thread, &arg[t]);
    }
    for (t = 0; t < threads; t++) {
        pthread_join(th[t], NULL);
        errors += arg[t].errors;
    }
    return errors;
}
