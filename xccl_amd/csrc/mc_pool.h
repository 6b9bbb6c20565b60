/*
 * mc_pool.h -- a cache of freed device blocks for the component's mem_alloc /
 * mem_free (vtable slots of reference src/utils/mem_component.h:30-31).
 *
 * The UCX team library allocates its scratch anew for every collective
 * (allreduce_knomial.c:181-183, reduce_knomial.c:120-121, allreduce_sra.c:177,
 * reduce_linear.c:78) and frees it at completion; the dispatcher's own cache
 * holds a single buffer of XCCL_MEM_COMPONENT_CACHE_SIZE (4 KiB by default,
 * mem_component.c:68-82), so anything larger costs a runtime allocation and a
 * runtime free -- which waits for the device -- per collective.  This cache
 * keeps freed blocks, by size class, up to a byte limit, and hands them out
 * again.
 *
 * The backing allocator is injected so that the bookkeeping can be exercised
 * without a device.  Thread-safe (one lock).  Not a general allocator: blocks
 * are never split or merged.
 */
#ifndef XCCL_ROCM_MC_POOL_H_
#define XCCL_ROCM_MC_POOL_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MC_POOL_MAX_BLOCKS 256

/* Both return 0 on success. */
typedef int (*mc_pool_backing_alloc_fn)(void **ptr, size_t len);
typedef int (*mc_pool_backing_free_fn)(void *ptr);

typedef struct mc_pool_stats {
    uint64_t hits;          /* allocations served from the cache */
    uint64_t misses;        /* allocations that went to the backing allocator */
    uint64_t backing_frees; /* blocks given back to the backing allocator */
    size_t   cached_bytes;  /* bytes held in free blocks right now */
    size_t   live_blocks;   /* blocks handed out and not yet freed */
    size_t   free_blocks;   /* blocks cached */
} mc_pool_stats_t;

/* Size class of a request: `len` rounded up to 4 KiB at least and then to the
 * next multiple of one eighth of its power of two (waste <= 12.5 %).  0 for
 * len == 0 and for requests too large to round. */
size_t mc_pool_size_class(size_t len);

/* (Re)configures the cache.  `limit_bytes` bounds the bytes kept in FREE
 * blocks; 0 turns caching off (every call goes to the backing allocator). */
void mc_pool_configure(mc_pool_backing_alloc_fn alloc_fn, mc_pool_backing_free_fn free_fn, size_t limit_bytes);

/* Changes the limit only; frees cached blocks beyond the new limit. */
void mc_pool_set_limit(size_t limit_bytes);

/* A block of at least `len` bytes for device ordinal `device`.
 * Returns what the backing allocator returned when it had to be asked. */
int mc_pool_alloc(int device, void **ptr, size_t len);

/* Takes back a block.  Blocks this cache does not know (allocated while
 * caching was off, or when its table was full) go straight to the backing
 * free. */
int mc_pool_free(void *ptr);

/* Gives every cached block back to the backing allocator (`device` < 0: all
 * devices).  Live blocks stay live and are forgotten when freed. */
void mc_pool_trim(int device);

void mc_pool_get_stats(mc_pool_stats_t *out);

#ifdef __cplusplus
}
#endif
#endif /* XCCL_ROCM_MC_POOL_H_ */
