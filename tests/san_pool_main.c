/* Runs the freed-block cache (xccl_amd/csrc/mc_pool.c) through its whole API
 * under a sanitizer: built by tests/test_sanitizers.py from this file,
 * tests/pool_harness.c and mc_pool.c with -fsanitize=address,undefined or
 * -fsanitize=thread, and run as a child process.  Exit status 0 = the
 * harness saw no error; the sanitizer reports its own findings and makes the
 * status non-zero.  Not a product file. */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "mc_pool.h"

void harness_configure(size_t limit);
long harness_stress(int threads, int iters);
long harness_backing_allocs(void);
long harness_backing_frees(void);
void harness_fail_next(int n);

#define CHECK(cond)                                                       \
    do {                                                                  \
        if (!(cond)) {                                                    \
            fprintf(stderr, "%s:%d: %s failed\n", __FILE__, __LINE__, #cond); \
            return 1;                                                     \
        }                                                                 \
    } while (0)

int main(int argc, char **argv)
{
    int             threads = argc > 1 ? atoi(argv[1]) : 8;
    int             iters   = argc > 2 ? atoi(argv[2]) : 20000;
    void           *p[MC_POOL_MAX_BLOCKS + 8];
    void           *q = NULL;
    mc_pool_stats_t st;
    int             i;

    /* hit / miss / reuse / limit / trim, single thread */
    harness_configure((size_t)1 << 20);
    CHECK(mc_pool_alloc(0, &p[0], 5000) == 0);
    memset(p[0], 1, 5000);
    CHECK(mc_pool_free(p[0]) == 0);
    CHECK(mc_pool_alloc(0, &q, 5100) == 0 && q == p[0]); /* same size class */
    CHECK(mc_pool_alloc(1, &p[1], 5100) == 0 && p[1] != q); /* other device */
    CHECK(mc_pool_free(q) == 0 && mc_pool_free(p[1]) == 0);
    CHECK(mc_pool_alloc(0, &p[2], (size_t)2 << 20) == 0); /* larger than the limit: never cached */
    CHECK(mc_pool_free(p[2]) == 0);
    mc_pool_get_stats(&st);
    CHECK(st.live_blocks == 0 && st.cached_bytes <= ((size_t)1 << 20));
    mc_pool_set_limit(4096); /* evicts down to the new limit */
    mc_pool_get_stats(&st);
    CHECK(st.cached_bytes <= 4096);
    mc_pool_trim(-1);
    mc_pool_get_stats(&st);
    CHECK(st.free_blocks == 0 && st.cached_bytes == 0);

    /* more live blocks than the table holds: the overflow goes straight to the backing allocator */
    harness_configure((size_t)64 << 20);
    for (i = 0; i < MC_POOL_MAX_BLOCKS + 8; i++) {
        CHECK(mc_pool_alloc(0, &p[i], 4096) == 0);
        memset(p[i], i, 4096);
    }
    for (i = 0; i < MC_POOL_MAX_BLOCKS + 8; i++) {
        CHECK(mc_pool_free(p[i]) == 0);
    }
    /* a failing backing allocator: the cache is emptied, the request retried once, then the error is passed on */
    harness_fail_next(1);
    CHECK(mc_pool_alloc(0, &q, (size_t)8 << 20) == 0);
    CHECK(mc_pool_free(q) == 0);
    harness_fail_next(2);
    CHECK(mc_pool_alloc(0, &q, (size_t)16 << 20) != 0);
    harness_fail_next(0);
    /* a pointer the cache never saw, and a zero-length request */
    q = malloc(100);
    CHECK(mc_pool_free(q) == 0);
    CHECK(mc_pool_alloc(0, &q, 0) == 0);
    CHECK(mc_pool_free(q) == 0);

    /* several threads, caching on and off */
    CHECK(harness_stress(threads, iters) == 0);
    harness_configure(0);
    CHECK(harness_stress(threads, iters / 4) == 0);
    harness_configure((size_t)8 << 20);
    CHECK(harness_stress(threads, iters) == 0);
    mc_pool_trim(-1);
    mc_pool_get_stats(&st);
    CHECK(st.live_blocks == 0 && st.free_blocks == 0);
    /* nothing leaked, nothing freed twice: every backing allocation was given back, plus the one foreign pointer */
    CHECK(harness_backing_allocs() + 1 == harness_backing_frees());
    printf("pool ok: %d threads x %d iterations, %ld backing allocations\n", threads, iters, harness_backing_allocs());
    return 0;
}
