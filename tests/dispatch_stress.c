/* Several threads borrowing and returning small buffers through the
 * dispatcher at once (libxccl_mc.so, a stand-in component loaded): the one
 * cached buffer must never be lent to two of them.  Built and run by
 * tests/test_abi.py.  Not a product file. */
#include <pthread.h>
#include <string.h>

#include "xccl_rocm_mem_component.h"

typedef struct {
    int  id, iters, mem_type;
    long errors, got_cached;
    void *cached;
} arg_t;

static void *worker(void *p)
{
    arg_t *a = (arg_t *)p;
    int    i;

    for (i = 0; i < a->iters; i++) {
        unsigned char *buf = NULL;
        size_t         j;
        if (xccl_mem_component_alloc((void **)&buf, 64, (ucs_memory_type_t)a->mem_type) != XCCL_OK || buf == NULL) {
            a->errors++;
            continue;
        }
        a->got_cached += (void *)buf == a->cached;
        memset(buf, a->id, 64);
        for (j = 0; j < 64; j++) {
            a->errors += buf[j] != (unsigned char)a->id; /* somebody else holds the same buffer */
        }
        if (xccl_mem_component_free(buf, (ucs_memory_type_t)a->mem_type) != XCCL_OK) {
            a->errors++;
        }
    }
    return NULL;
}

/* Returns the number of corrupted bytes and failed calls over all threads;
 * *cached_loans receives how often the cached buffer was the one lent. */
long dispatch_stress(int threads, int iters, int mem_type, long *cached_loans)
{
    pthread_t th[16];
    arg_t     arg[16];
    void     *first = NULL;
    long      errors = 0;
    int       t;

    if (threads > 16) {
        threads = 16;
    }
    /* the first small request creates the cached buffer; remember which it is */
    if (xccl_mem_component_alloc(&first, 64, (ucs_memory_type_t)mem_type) != XCCL_OK) {
        return -1;
    }
    xccl_mem_component_free(first, (ucs_memory_type_t)mem_type);
    for (t = 0; t < threads; t++) {
        arg[t] = (arg_t){.id = t + 1, .iters = iters, .mem_type = mem_type, .cached = first};
        pthread_create(&th[t], NULL, worker, &arg[t]);
    }
    *cached_loans = 0;
    for (t = 0; t < threads; t++) {
        pthread_join(th[t], NULL);
        errors += arg[t].errors;
        *cached_loans += arg[t].got_cached;
    }
    return errors;
}
