/*
 * xccl_rocm_mem_pool.h -- knobs of the freed-block cache behind the ROCm
 * memory component's mem_alloc / mem_free (vtable slots of reference
 * src/utils/mem_component.h:30-31; reference implementation
 * src/utils/cuda/cuda_mem_component.c:34-44 is a bare cudaMalloc / cudaFree).
 *
 * The UCX team library allocates scratch per collective and frees it at
 * completion (allreduce_knomial.c:181-183, reduce_knomial.c:120-121,
 * allreduce_sra.c:177, reduce_linear.c:78); beyond the dispatcher's single
 * small cached buffer (mem_component.c:68-82) each of those is a runtime
 * allocation plus a runtime free that waits for the device.  The component
 * keeps freed blocks by size class (request rounded up to 4 KiB at least, then
 * to an eighth-of-a-power-of-two step: at most 12.5 % over-allocation) and
 * hands them out again.  A block returned by mem_free is reusable at once,
 * and -- unlike the reference's cudaFree -- mem_free does not wait for the
 * device: free a block only after every stream-ordered reduction, copy or
 * kernel that touches it has completed (event_query / event_wait say when),
 * or another thread's mem_alloc may receive it while that work still runs.
 *
 * The limit is the number of bytes that may sit in FREE blocks; least recently
 * freed blocks are released first.  Default 8 GiB, or the environment variable
 * XCCL_MC_ROCM_POOL_MAX_BYTES (read in open()); 0 turns the cache off, and
 * mem_alloc / mem_free are then the runtime's calls, as in the reference.
 * Exported by xccl_rocm_mem_component.so.  No counterpart in the reference.
 */
#ifndef XCCL_ROCM_MEM_POOL_H_
#define XCCL_ROCM_MEM_POOL_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct xccl_rocm_mem_pool_stats {
    uint64_t hits;          /* mem_alloc calls served from cached blocks */
    uint64_t misses;        /* mem_alloc calls that reached the runtime allocator */
    uint64_t backing_frees; /* blocks released to the runtime */
    size_t   cached_bytes;  /* bytes in free blocks now */
    size_t   live_blocks;   /* tracked blocks handed out */
    size_t   free_blocks;   /* blocks cached */
} xccl_rocm_mem_pool_stats_t;

/* Sets the limit; releases cached blocks beyond it (0: release all, stop caching). */
void xccl_rocm_mem_pool_set_limit(size_t limit_bytes);

void xccl_rocm_mem_pool_get_stats(xccl_rocm_mem_pool_stats_t *out);

#ifdef __cplusplus
}
#endif
#endif /* XCCL_ROCM_MEM_POOL_H_ */
