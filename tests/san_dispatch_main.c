/* Runs the dispatcher (xccl_amd/csrc/mc_dispatch.c) under a sanitizer with
 * the host-memory stand-in component (tests/fake_component.c) loaded: the
 * loader, every forwarding entry, the stream-ordered entries' fallback rule,
 * then several threads borrowing the cached buffer at once
 * (tests/dispatch_stress.c).  Built by tests/test_sanitizers.py with
 * -fsanitize=address,undefined or -fsanitize=thread and run as a child
 * process: argv[1] is the directory that holds the stand-in component as
 * xccl_cuda_mem_component.so (plain vtable) and xccl_rocm_mem_component.so
 * (with the extension).  Not a product file. */
#include <stdio.h>
#include <stdlib.h>

#include "xccl_rocm_mem_component.h"

long dispatch_stress(int threads, int iters, int mem_type, long *cached_loans);

#define CHECK(cond)                                                       \
    do {                                                                  \
        if (!(cond)) {                                                    \
            fprintf(stderr, "%s:%d: %s failed\n", __FILE__, __LINE__, #cond); \
            return 1;                                                     \
        }                                                                 \
    } while (0)

int main(int argc, char **argv)
{
    int                                  threads = argc > 2 ? atoi(argv[2]) : 8;
    int                                  iters   = argc > 3 ? atoi(argv[3]) : 50000;
    void                                *hip_stream = (void *)0x1234;
    xccl_stream_t                        s      = {XCCL_STREAM_TYPE_ROCM, &hip_stream};
    xccl_stream_t                        bad    = {(xccl_stream_type_t)7, &hip_stream};
    xccl_mc_event_t                     *ev     = NULL;
    xccl_mem_component_stream_request_t *req    = NULL;
    ucs_memory_type_t                    mt;
    char                                 src[32] = "0123456789abcdef", dst[32];
    void                                *p = NULL, *q = NULL;
    long                                 loans = 0;

    CHECK(argc > 1);
    CHECK(xccl_mem_component_init(NULL) == XCCL_ERR_INVALID_PARAM);
    CHECK(xccl_mem_component_init(argv[1]) == XCCL_OK);
    CHECK(xccl_mem_component_init(argv[1]) == XCCL_OK); /* a second init keeps what is loaded */
    CHECK(xccl_mem_component_get(UCS_MEMORY_TYPE_CUDA) != NULL && xccl_mem_component_get(UCS_MEMORY_TYPE_ROCM) != NULL);
    CHECK(xccl_mem_component_get(UCS_MEMORY_TYPE_HOST) == NULL && xccl_mem_component_get((ucs_memory_type_t)99) == NULL);

    CHECK(xccl_mem_component_alloc(&p, 100, UCS_MEMORY_TYPE_ROCM) == XCCL_OK);
    CHECK(xccl_mem_component_alloc(&q, 100000, UCS_MEMORY_TYPE_ROCM) == XCCL_OK);
    CHECK(xccl_mem_component_type(src, &mt) == XCCL_OK && mt == UCS_MEMORY_TYPE_HOST);
    CHECK(xccl_mem_component_reduce(src, src, dst, 4, XCCL_DT_INT32, XCCL_OP_SUM, UCS_MEMORY_TYPE_ROCM) == XCCL_OK);
    CHECK(xccl_mem_component_reduce(src, src, dst, 4, XCCL_DT_INT32, XCCL_OP_SUM, UCS_MEMORY_TYPE_HOST) ==
          XCCL_ERR_UNSUPPORTED);
    CHECK(xccl_mem_component_reduce_multi(src, src, dst, 2, 0, 16, XCCL_DT_INT32, XCCL_OP_SUM,
                                          UCS_MEMORY_TYPE_ROCM_MANAGED) == XCCL_OK);
    CHECK(xccl_mem_component_reduce_multi(src, src, dst, 2, 4, 16, XCCL_DT_INT32, XCCL_OP_SUM,
                                          UCS_MEMORY_TYPE_ROCM_MANAGED) == XCCL_ERR_UNSUPPORTED);
    /* stream-ordered entries: with and without the extension, with and without a stream and an event */
    CHECK(xccl_mem_component_reduce_multi_nb(src, src, dst, 2, 4, 16, XCCL_DT_INT32, XCCL_OP_SUM, UCS_MEMORY_TYPE_ROCM,
                                             NULL, &ev) == XCCL_OK && ev != NULL && ev->mem_type == UCS_MEMORY_TYPE_ROCM);
    CHECK(xccl_mc_event_query(ev) == XCCL_INPROGRESS && xccl_mc_event_wait(ev) == XCCL_OK && xccl_mc_event_free(ev) == XCCL_OK);
    CHECK(xccl_mem_component_reduce_nb(src, src, dst, 4, XCCL_DT_INT32, XCCL_OP_SUM, UCS_MEMORY_TYPE_ROCM, &s, NULL) == XCCL_OK);
    CHECK(xccl_mem_component_reduce_nb(src, src, dst, 0, XCCL_DT_INT32, XCCL_OP_SUM, UCS_MEMORY_TYPE_ROCM, NULL, &ev) ==
          XCCL_OK && ev == NULL);
    CHECK(xccl_mem_component_reduce_nb(src, src, dst, 4, XCCL_DT_INT32, XCCL_OP_SUM, UCS_MEMORY_TYPE_CUDA, NULL, &ev) ==
          XCCL_OK && ev == NULL);
    CHECK(xccl_mem_component_reduce_multi_nb(src, src, dst, 2, 4, 16, XCCL_DT_INT32, XCCL_OP_SUM, UCS_MEMORY_TYPE_CUDA,
                                             &s, &ev) == XCCL_ERR_NOT_IMPLEMENTED);
    CHECK(xccl_mem_component_reduce_nb(src, src, dst, 4, XCCL_DT_INT32, XCCL_OP_SUM, UCS_MEMORY_TYPE_HOST, NULL, NULL) ==
          XCCL_ERR_UNSUPPORTED);
    /* entries routed by the stream's type */
    CHECK(xccl_mc_event_record(&s, &ev) == XCCL_OK && ev->mem_type == UCS_MEMORY_TYPE_ROCM);
    CHECK(xccl_mc_event_free(ev) == XCCL_OK);
    CHECK(xccl_mc_event_record(&bad, &ev) == XCCL_ERR_UNSUPPORTED && xccl_mc_event_record(NULL, &ev) == XCCL_ERR_UNSUPPORTED);
    CHECK(xccl_mc_event_query(NULL) == XCCL_ERR_UNSUPPORTED && xccl_mc_event_wait(NULL) == XCCL_ERR_UNSUPPORTED);
    CHECK(xccl_mem_component_memcpy_async(src, dst, 16, &s) == XCCL_OK && dst[15] == 'f');
    CHECK(xccl_mem_component_memcpy_async(src, dst, 0, NULL) == XCCL_OK);
    CHECK(xccl_mem_component_start_acitivity(&s, &req) == XCCL_OK && req->mem_type == UCS_MEMORY_TYPE_ROCM);
    CHECK(xccl_mem_component_finish_acitivity(req) == XCCL_OK && xccl_mem_component_finish_acitivity(NULL) == XCCL_ERR_UNSUPPORTED);
    CHECK(xccl_mem_component_free(p, UCS_MEMORY_TYPE_ROCM) == XCCL_OK && xccl_mem_component_free(q, UCS_MEMORY_TYPE_ROCM) == XCCL_OK);

    /* the cached buffer under contention, on both components */
    CHECK(dispatch_stress(threads, iters, UCS_MEMORY_TYPE_ROCM, &loans) == 0 && loans > 0);
    CHECK(dispatch_stress(threads, iters, UCS_MEMORY_TYPE_CUDA, &loans) == 0 && loans > 0);

    xccl_mem_component_free_cache();
    xccl_mem_component_finalize();
    CHECK(xccl_mem_component_get(UCS_MEMORY_TYPE_ROCM) == NULL);
    printf("dispatch ok: %d threads x %d iterations\n", threads, iters);
    return 0;
}
