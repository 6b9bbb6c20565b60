/* The two objects the reference's src/utils/mem_component.c takes from the
 * rest of libxccl and from UCX, defined here so that this one file can be
 * built into a shared object of its own (tests/refdispatch/Makefile):
 *   xccl_lib_global_config   reference src/core/xccl_global_opts.c:3-8
 *                            (cache size 4096 by default; log level WARN)
 *   ucs_memory_type_names[]  UCX v1.10 ucs/memory/memory_type.c
 * Test infrastructure: nothing in the product links this. */
#include <stdlib.h>

#include "utils/xccl_log.h"
#include <ucs/memory/memory_type.h>

xccl_config_t xccl_lib_global_config = {
    .log_component            = {UCS_LOG_LEVEL_WARN, "XCCL"},
    .team_lib_path            = NULL,
    .mem_component_cache_size = 4096,
    .lf_tasks_queue_size      = 8,
};

const char *ucs_memory_type_names[] = {
    [UCS_MEMORY_TYPE_HOST]         = "host",
    [UCS_MEMORY_TYPE_CUDA]         = "cuda",
    [UCS_MEMORY_TYPE_CUDA_MANAGED] = "cuda-managed",
    [UCS_MEMORY_TYPE_ROCM]         = "rocm",
    [UCS_MEMORY_TYPE_ROCM_MANAGED] = "rocm-managed",
    [UCS_MEMORY_TYPE_LAST]         = "unknown",
};

/* what libxccl's option parser would do with XCCL_MEM_COMPONENT_CACHE_SIZE */
__attribute__((constructor)) static void ref_globals_from_env(void)
{
    const char *v = getenv("XCCL_MEM_COMPONENT_CACHE_SIZE");

    if (v != NULL) {
        xccl_lib_global_config.mem_component_cache_size = (size_t)strtoull(v, NULL, 0);
    }
}
