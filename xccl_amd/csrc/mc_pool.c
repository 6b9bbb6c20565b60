/*
 * mc_pool.c -- bookkeeping of the freed-block cache described in mc_pool.h.
 * No device call in here: the backing allocator is whatever the component
 * configured (the HIP runtime's allocator in production, the C library's in
 * the host-only tests).
 */
#include "mc_pool.h"

#include <pthread.h>
#include <string.h>

enum { SLOT_EMPTY = 0, SLOT_LIVE = 1, SLOT_FREE = 2 };

typedef struct mc_pool_slot {
    void    *ptr;
    size_t   bytes;  /* size class the block was allocated with */
    int      device;
    int      state;
    uint64_t stamp;  /* when it was freed (eviction order) */
} mc_pool_slot_t;

static struct {
    pthread_mutex_t          lock;
    mc_pool_slot_t           slot[MC_POOL_MAX_BLOCKS];
    mc_pool_backing_alloc_fn alloc_fn;
    mc_pool_backing_free_fn  free_fn;
    size_t                   limit;
    size_t                   cached_bytes;
    uint64_t                 clock;
    uint64_t                 hits, misses, backing_frees;
} pool = {.lock = PTHREAD_MUTEX_INITIALIZER};

size_t mc_pool_size_class(size_t len)
{
    size_t pow2, step;

    if (len == 0 || len > ((size_t)1 << 62)) {
        return 0;
    }
    if (len <= 4096) {
        return 4096;
    }
    pow2 = 4096;
    while (pow2 < len) {
        pow2 <<= 1;
    }
    step = pow2 >> 4; /* classes every eighth of the way from pow2/2 to pow2 */
    return (len + step - 1) / step * step;
}

/* Detaches cached blocks, oldest first, until at most `limit` bytes stay
 * cached; the detached pointers go to out[] for the caller to free once the
 * lock is dropped.  Lock held. */
static size_t evict_down_to(size_t limit, void **out)
{
    size_t n = 0;

    while (pool.cached_bytes > limit) {
        mc_pool_slot_t *oldest = NULL;
        int             i;
        for (i = 0; i < MC_POOL_MAX_BLOCKS; i++) {
            mc_pool_slot_t *s = &pool.slot[i];
            if (s->state == SLOT_FREE && (oldest == NULL || s->stamp < oldest->stamp)) {
                oldest = s;
            }
        }
        if (oldest == NULL) {
            pool.cached_bytes = 0; /* nothing cached: the count was stale */
            break;
        }
        out[n++] = oldest->ptr;
        pool.cached_bytes -= oldest->bytes;
        memset(oldest, 0, sizeof(*oldest));
    }
    return n;
}

static void backing_free_all(void **ptrs, size_t n)
{
    size_t i;

    for (i = 0; i < n; i++) {
        (void)pool.free_fn(ptrs[i]);
    }
    if (n > 0) {
        pthread_mutex_lock(&pool.lock);
        pool.backing_frees += n;
        pthread_mutex_unlock(&pool.lock);
    }
}

void mc_pool_configure(mc_pool_backing_alloc_fn alloc_fn, mc_pool_backing_free_fn free_fn, size_t limit_bytes)
{
    pthread_mutex_lock(&pool.lock);
    pool.alloc_fn = alloc_fn;
    pool.free_fn  = free_fn;
    pthread_mutex_unlock(&pool.lock);
    mc_pool_set_limit(limit_bytes);
}

void mc_pool_set_limit(size_t limit_bytes)
{
    void  *victims[MC_POOL_MAX_BLOCKS];
    size_t n;

    pthread_mutex_lock(&pool.lock);
    pool.limit = limit_bytes;
    n          = evict_down_to(limit_bytes, victims);
    pthread_mutex_unlock(&pool.lock);
    backing_free_all(victims, n);
}

int mc_pool_alloc(int device, void **ptr, size_t len)
{
    const size_t cls = mc_pool_size_class(len);
    int          i, rc;

    pthread_mutex_lock(&pool.lock);
    if (cls == 0 || pool.limit == 0) {
        pthread_mutex_unlock(&pool.lock);
        return pool.alloc_fn(ptr, len); /* not tracked */
    }
    for (i = 0; i < MC_POOL_MAX_BLOCKS; i++) {
        mc_pool_slot_t *s = &pool.slot[i];
        if (s->state == SLOT_FREE && s->device == device && s->bytes == cls) {
            s->state = SLOT_LIVE;
            pool.cached_bytes -= cls;
            pool.hits++;
            *ptr = s->ptr;
            pthread_mutex_unlock(&pool.lock);
            return 0;
        }
    }
    pool.misses++;
    pthread_mutex_unlock(&pool.lock);

    rc = pool.alloc_fn(ptr, cls);
    if (rc != 0) {
        /* the cache itself may be what fills the device: empty it, try once more */
        mc_pool_trim(-1);
        rc = pool.alloc_fn(ptr, cls);
        if (rc != 0) {
            return rc;
        }
    }
    pthread_mutex_lock(&pool.lock);
    for (i = 0; i < MC_POOL_MAX_BLOCKS; i++) {
        mc_pool_slot_t *s = &pool.slot[i];
        if (s->state == SLOT_EMPTY) {
            s->ptr    = *ptr;
            s->bytes  = cls;
            s->device = device;
            s->state  = SLOT_LIVE;
            break;
        }
    } /* table full: the block stays untracked and its free goes to the backing allocator */
    pthread_mutex_unlock(&pool.lock);
    return 0;
}

int mc_pool_free(void *ptr)
{
    void           *victims[MC_POOL_MAX_BLOCKS];
    size_t          n = 0;
    mc_pool_slot_t *s = NULL;
    int             i;

    if (ptr == NULL) {
        return 0;
    }
    pthread_mutex_lock(&pool.lock);
    for (i = 0; i < MC_POOL_MAX_BLOCKS; i++) {
        if (pool.slot[i].state != SLOT_EMPTY && pool.slot[i].ptr == ptr) {
            s = &pool.slot[i];
            break;
        }
    }
    if (s == NULL) {
        pthread_mutex_unlock(&pool.lock);
        return pool.free_fn(ptr); /* not ours to cache */
    }
    if (s->state == SLOT_FREE) {
        pthread_mutex_unlock(&pool.lock);
        return -1; /* freed twice */
    }
    if (s->bytes > pool.limit) {
        memset(s, 0, sizeof(*s));
        victims[n++] = ptr;
    } else {
        s->state = SLOT_FREE;
        s->stamp = ++pool.clock;
        pool.cached_bytes += s->bytes;
        n = evict_down_to(pool.limit, victims);
    }
    pthread_mutex_unlock(&pool.lock);
    backing_free_all(victims, n);
    return 0;
}

void mc_pool_trim(int device)
{
    void  *victims[MC_POOL_MAX_BLOCKS];
    size_t n = 0;
    int    i;

    pthread_mutex_lock(&pool.lock);
    for (i = 0; i < MC_POOL_MAX_BLOCKS; i++) {
        mc_pool_slot_t *s = &pool.slot[i];
        if (s->state == SLOT_FREE && (device < 0 || s->device == device)) {
            victims[n++] = s->ptr;
            pool.cached_bytes -= s->bytes;
            memset(s, 0, sizeof(*s));
        }
    }
    pthread_mutex_unlock(&pool.lock);
    backing_free_all(victims, n);
}

void mc_pool_get_stats(mc_pool_stats_t *out)
{
    int i;

    memset(out, 0, sizeof(*out));
    pthread_mutex_lock(&pool.lock);
    out->hits          = pool.hits;
    out->misses        = pool.misses;
    out->backing_frees = pool.backing_frees;
    out->cached_bytes  = pool.cached_bytes;
    for (i = 0; i < MC_POOL_MAX_BLOCKS; i++) {
        out->live_blocks += pool.slot[i].state == SLOT_LIVE;
        out->free_blocks += pool.slot[i].state == SLOT_FREE;
    }
    pthread_mutex_unlock(&pool.lock);
}
