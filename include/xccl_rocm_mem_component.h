/*
 * xccl_rocm_mem_component.h -- the plugin boundary of the ROCm memory
 * component, and the dispatcher that drives it.
 *
 * 1. xccl_mem_component_t is XCCL's memory-component vtable (reference
 *    src/utils/mem_component.h:28-49), member for member.  libxccl dlopens
 *    `<plugin dir>/xccl_<memtype>_mem_component.so`, looks up ONE data symbol
 *    whose first member is this struct, and calls through it (reference
 *    src/utils/mem_component.c:11-49).
 *
 * 2. xccl_rocm_mem_component_t is the object xccl_rocm_mem_component.so
 *    exports, under two names: `xccl_rocm_mem_component`, and the alias
 *    `xccl_cuda_mem_component` because the reference loader looks up that
 *    literal name for every memory type (mem_component.c:30).  It extends the
 *    vtable at its tail with stream-ordered reductions and event completion
 *    for the UCX team library's k-nomial / scatter-reduce call sites
 *    (reference src/team_lib/ucx/allreduce/allreduce_knomial.c:129-135,
 *    allreduce_sra.c:281-284, reduce/reduce_knomial.c:79-85).
 *
 * 3. xccl_mem_component_*() is the dispatcher libxccl keeps in
 *    src/utils/mem_component.c, restated in libxccl_mc.so so that the
 *    component can be loaded and driven without libxccl and UCX.  Same names,
 *    arguments and status codes.  One deliberate difference: this dispatcher
 *    does no arithmetic itself, so reduce / reduce_multi on
 *    UCS_MEMORY_TYPE_HOST return XCCL_ERR_UNSUPPORTED here (in libxccl that
 *    branch is the inline CPU loop of src/utils/reduce.h and is untouched by
 *    this component).
 */
#ifndef XCCL_ROCM_MEM_COMPONENT_H_
#define XCCL_ROCM_MEM_COMPONENT_H_

#include "xccl_rocm_types.h"

#ifdef XCCL_MC_ROCM_IN_TREE
#include <utils/mem_component.h>
#else

#ifdef __cplusplus
extern "C" {
#endif

/* reference src/utils/mem_component.h:13-26 */
typedef struct xccl_mem_component_buf {
    void  *buf;
    size_t size;
    int    used;
} xccl_mem_component_buf_t;

typedef struct xccl_mem_component_stream_request {
    ucs_memory_type_t mem_type;
} xccl_mem_component_stream_request_t;

typedef struct xccl_mc_event {
    ucs_memory_type_t mem_type;
} xccl_mc_event_t;

/* reference src/utils/mem_component.h:28-49 -- order and signatures fixed */
typedef struct xccl_mem_component {
    xccl_status_t (*open)(void);
    xccl_status_t (*mem_alloc)(void **ptr, size_t len);
    xccl_status_t (*mem_free)(void *ptr);
    xccl_status_t (*mem_type)(void *ptr, ucs_memory_type_t *mem_type);
    xccl_status_t (*reduce)(void *sbuf1, void *sbuf2, void *target,
                            size_t count, xccl_dt_t dtype, xccl_op_t op);
    xccl_status_t (*reduce_multi)(void *sbuf1, void *sbuf2, void *rbuf,
                                  size_t count, size_t size, size_t stride,
                                  xccl_dt_t dtype, xccl_op_t op);
    xccl_status_t (*memcpy_async)(void *sbuf, void *dbuf, size_t size,
                                  xccl_stream_t *stream);
    xccl_status_t (*event_record)(xccl_stream_t *stream,
                                  xccl_mc_event_t **event);
    xccl_status_t (*event_query)(xccl_mc_event_t *event);
    xccl_status_t (*event_free)(xccl_mc_event_t *event);
    xccl_status_t (*start_stream_activity)(
        xccl_stream_t *stream, xccl_mem_component_stream_request_t **req);
    xccl_status_t (*finish_stream_activity)(
        xccl_mem_component_stream_request_t *req);
    void (*close)(void);
    void                    *dlhandle; /* written by the loader */
    xccl_mem_component_buf_t cache;    /* written by the loader */
} xccl_mem_component_t;

#ifdef __cplusplus
}
#endif
#endif /* XCCL_MC_ROCM_IN_TREE */

#ifdef __cplusplus
extern "C" {
#endif

#define XCCL_ROCM_MC_EXT_VERSION 1u
#define XCCL_ROCM_MC_NUM_EVENTS 64          /* reference pool: 4 */
#define XCCL_ROCM_MC_NUM_STREAM_REQUESTS 4  /* reference pool: 4 */

/*
 * Exported object.  `super` is what an unmodified libxccl sees.  The members
 * after it are the extension; a caller that knows them checks `ext_version`.
 *
 * reduce_nb / reduce_multi_nb: same arithmetic contract as reduce /
 * reduce_multi, but the call returns once the kernel is enqueued.
 *   stream == NULL : enqueue on the component's queue of the CALLING THREAD
 *                    (the one the synchronous entries use on that thread), so
 *                    successive calls of one thread are ordered among
 *                    themselves.  That queue is a HIP stream (get_stream) for
 *                    calls without an event; a call that has an event goes out
 *                    on a dispatch queue of the component's own instead when
 *                    the stream holds nothing it would have to stay behind
 *                    (4.6-6.0 us per small call instead of 6.8-7.8;
 *                    XCCL_MC_ROCM_DIRECT_QUEUE=0 switches that off).  The
 *                    order of one thread's calls holds across the two; only
 *                    the event tells when such a call is complete.  Threads
 *                    are spread round-robin over up to 4 streams per device
 *                    (XCCL_MC_ROCM_THREAD_STREAMS, 1..4), so that blocking
 *                    calls of several threads (XCCL_THREAD_MODE_MULTIPLE) do
 *                    not queue up behind each other's kernels; calls of
 *                    different threads are not ordered among themselves;
 *   stream != NULL : enqueue on *(hipStream_t*)stream->stream.
 *   event  != NULL : *event receives a pooled event recorded right after the
 *                    kernel; poll it with event_query (XCCL_INPROGRESS /
 *                    XCCL_OK), block on it with event_wait, return it with
 *                    event_free.  XCCL_ERR_NO_RESOURCE when the pool is empty
 *                    (nothing is enqueued then).
 * With event == NULL the entries do nothing but enqueue one kernel, so a
 * caller may record them into its own hipGraph through stream capture; an
 * event must not be requested while capturing (its completion is tied to
 * this one launch, not to later replays).  The component creates its
 * per-device resources on the first call on a device, which allocates and
 * synchronises: make that call outside any capture (a call with a capturing
 * `stream` on a device not yet used returns XCCL_ERR_NO_RESOURCE, from these
 * entries as from event_record and start_stream_activity).
 *
 * finish_stream_activity returns XCCL_ERR_NO_PROGRESS when the gate kernel
 * had already given up (XCCL_MC_ROCM_GATE_TIMEOUT_MS, default 30 s; the
 * reference kernel spins without a bound): work queued behind the gate then
 * ran before the collective finished, and the caller must not trust stream
 * order for it.
 *
 * mem_free keeps the block for the next mem_alloc and does not wait for the
 * device (the reference's cudaFree does): free a block only after all work
 * that touches it has completed.
 * These replace the launch + cudaStreamSynchronize pair of the reference
 * (xccl_cuda_reduce_multi.cu:42-44,140) at the call sites named above.
 */
typedef struct xccl_rocm_mem_component {
    xccl_mem_component_t super;
    uint32_t             ext_version;
    xccl_status_t (*reduce_nb)(void *sbuf1, void *sbuf2, void *target,
                               size_t count, xccl_dt_t dtype, xccl_op_t op,
                               xccl_stream_t *stream, xccl_mc_event_t **event);
    xccl_status_t (*reduce_multi_nb)(void *sbuf1, void *sbuf2, void *rbuf,
                                     size_t count, size_t size, size_t stride,
                                     xccl_dt_t dtype, xccl_op_t op,
                                     xccl_stream_t *stream,
                                     xccl_mc_event_t **event);
    xccl_status_t (*event_wait)(xccl_mc_event_t *event);
    /* The component's hipStream_t for the calling thread on the current
     * device (created on first use), as void*.  For callers that time or
     * order work against it: calls of that thread with stream == NULL and
     * event == NULL are on it; calls with an event may not be (above). */
    xccl_status_t (*get_stream)(void **hip_stream);
} xccl_rocm_mem_component_t;

/* Defined by xccl_rocm_mem_component.so; xccl_cuda_mem_component is an alias
 * of the same object.  xccl_rocm_mem_component_ext points at it: a loader
 * that wants the extension looks THAT symbol up
 * (xccl_<memory type name>_mem_component_ext), so it never has to read behind
 * the vtable of a component that may not have one. */
extern xccl_rocm_mem_component_t        xccl_rocm_mem_component;
extern xccl_rocm_mem_component_t *const xccl_rocm_mem_component_ext;

/* ------------------------------------------------------------------------
 * Dispatcher (libxccl_mc.so) -- reference src/utils/mem_component.h:52-95,
 * src/utils/mem_component.c.  `mem_type` arguments are ucs_memory_type_t.
 * ---------------------------------------------------------------------- */

/* mem_component.c:11-49.  Tries `<path>/xccl_<name>_mem_component.so` for
 * every non-host memory type (names host, cuda, cuda-managed, rocm,
 * rocm-managed).  The data symbol is looked up as `xccl_<name>_mem_component`
 * ('-' -> '_') first and as `xccl_cuda_mem_component` second; a file that
 * exports neither is skipped (the reference dereferences NULL there).  The
 * extension is taken from `xccl_<name>_mem_component_ext` if the file has it.
 * Cache size comes from XCCL_MEM_COMPONENT_CACHE_SIZE (default 4096,
 * reference src/core/xccl_global_opts.c:3-37). */
xccl_status_t xccl_mem_component_init(const char *components_path);

/* mem_component.c:51-105 (single cached buffer per component) */
xccl_status_t xccl_mem_component_alloc(void **ptr, size_t len,
                                       ucs_memory_type_t mem_type);
xccl_status_t xccl_mem_component_free(void *ptr, ucs_memory_type_t mem_type);

/* mem_component.c:150-174 */
xccl_status_t xccl_mem_component_type(void *ptr, ucs_memory_type_t *mem_type);

/* mem_component.c:107-120 */
xccl_status_t xccl_mem_component_reduce(void *sbuf1, void *sbuf2, void *target,
                                        size_t count, xccl_dt_t dtype,
                                        xccl_op_t op,
                                        ucs_memory_type_t mem_type);

/* mem_component.c:122-148; size == 0 is XCCL_OK without touching anything */
xccl_status_t xccl_mem_component_reduce_multi(void *sbuf1, void *sbuf2,
                                              void *rbuf, size_t count,
                                              size_t size, size_t stride,
                                              xccl_dt_t dtype, xccl_op_t op,
                                              ucs_memory_type_t mem_type);

/* Stream-ordered forms: the two entries integration/xccl-rocm.patch adds to
 * the reference's src/utils/mem_component.{h,c}, with the same arguments and
 * the same rule (an in-tree build, -DXCCL_MC_ROCM_IN_TREE, sees both
 * declarations and fails on any difference).  What the patched call sites of
 * the UCX team library call (allreduce_knomial.c:74-80,129-135,
 * allreduce_sra.c:212-218,281-284, reduce_knomial.c:79-85,
 * reduce_linear.c:28-34), always with stream == NULL.
 *   stream == NULL : the component's queue of the calling thread
 *   event  != NULL : *event is NULL when the reduction is complete on return,
 *                    else an event for xccl_mc_event_query / _free
 * Fallbacks, in this order: host memory or no component -> whatever the
 * blocking entry above returns; component without the extension -> the
 * blocking entry if stream == NULL, else XCCL_ERR_NOT_IMPLEMENTED; empty
 * reduction -> XCCL_OK; the component's event pool is empty
 * (XCCL_ERR_NO_RESOURCE, nothing enqueued) -> the blocking entry if
 * stream == NULL, else that error. */
xccl_status_t xccl_mem_component_reduce_nb(void *sbuf1, void *sbuf2,
                                           void *target, size_t count,
                                           xccl_dt_t dtype, xccl_op_t op,
                                           ucs_memory_type_t mem_type,
                                           xccl_stream_t *stream,
                                           xccl_mc_event_t **event);
xccl_status_t xccl_mem_component_reduce_multi_nb(
    void *sbuf1, void *sbuf2, void *rbuf, size_t count, size_t size,
    size_t stride, xccl_dt_t dtype, xccl_op_t op, ucs_memory_type_t mem_type,
    xccl_stream_t *stream, xccl_mc_event_t **event);

/* mem_component.c:180-229 (names keep the reference's spelling) */
xccl_status_t xccl_mem_component_memcpy_async(void *sbuf, void *dbuf,
                                              size_t size,
                                              xccl_stream_t *stream);
xccl_status_t xccl_mem_component_start_acitivity(
    xccl_stream_t *stream, xccl_mem_component_stream_request_t **req);
xccl_status_t xccl_mem_component_finish_acitivity(
    xccl_mem_component_stream_request_t *req);

/* mem_component.c:231-257 */
xccl_status_t xccl_mc_event_record(xccl_stream_t *stream,
                                   xccl_mc_event_t **event);
xccl_status_t xccl_mc_event_query(xccl_mc_event_t *event);
xccl_status_t xccl_mc_event_free(xccl_mc_event_t *event);
xccl_status_t xccl_mc_event_wait(xccl_mc_event_t *event); /* extension */

/* mem_component.c:259-283 */
void xccl_mem_component_free_cache(void);
void xccl_mem_component_finalize(void);

/* The loaded component for a memory type, or NULL (test/diagnostic hook). */
xccl_mem_component_t *xccl_mem_component_get(ucs_memory_type_t mem_type);

#ifdef __cplusplus
}
#endif
#endif /* XCCL_ROCM_MEM_COMPONENT_H_ */
