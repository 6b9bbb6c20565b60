/*
 * mc_dispatch.c -- libxccl_mc.so: XCCL's memory-component dispatcher,
 * restated so that a component can be loaded and driven without libxccl and
 * UCX.  Follows reference src/utils/mem_component.c function by function
 * (line ranges at each function); same names, arguments and status codes.
 *
 * Differences, all deliberate:
 *   - no arithmetic lives here: reduce / reduce_multi on HOST memory return
 *     XCCL_ERR_UNSUPPORTED (libxccl runs src/utils/reduce.h inline there);
 *   - the loader looks the component up by its own name before the
 *     hard-coded "xccl_cuda_mem_component" and skips a file exporting neither
 *     (mem_component.c:30 dereferences a NULL dlsym result);
 *   - stream_to_mem_type knows XCCL_STREAM_TYPE_ROCM (mem_component.c:176-178
 *     has the CUDA entry only);
 *   - the cached buffer is claimed atomically (mem_component.c:68-82 tests and
 *     sets `used` without synchronisation although collectives may be posted
 *     from several threads);
 *   - the *_nb entries are the ones integration/xccl-rocm.patch adds to the
 *     reference's dispatcher (same arguments, same fallback rule);
 *     xccl_mc_event_wait and xccl_mem_component_get exist only here.
 */
#include "xccl_rocm_mem_component.h"

#include <dlfcn.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static xccl_mem_component_t      *mem_components[UCS_MEMORY_TYPE_LAST];
static xccl_rocm_mem_component_t *mem_extensions[UCS_MEMORY_TYPE_LAST]; /* NULL: plain reference vtable */

/* UCX v1.10 ucs_memory_type_names[], indexed by ucs_memory_type_t */
static const char *const memory_type_names[UCS_MEMORY_TYPE_LAST] = {
    "host", "cuda", "cuda-managed", "rocm", "rocm-managed"
};

static const ucs_memory_type_t stream_to_mem_type[XCCL_STREAM_TYPE_LAST] = {
    [XCCL_STREAM_TYPE_CUDA] = UCS_MEMORY_TYPE_CUDA,
    [XCCL_STREAM_TYPE_ROCM] = UCS_MEMORY_TYPE_ROCM,
};

static xccl_mem_component_t *component_of(int mt)
{
    if (mt <= UCS_MEMORY_TYPE_HOST || mt >= UCS_MEMORY_TYPE_LAST) {
        return NULL;
    }
    return mem_components[mt];
}

/* The stream-ordered extension of the component loaded for `mt`, or NULL. */
static xccl_rocm_mem_component_t *extension_of(int mt)
{
    return component_of(mt) ? mem_extensions[mt] : NULL;
}

static xccl_mem_component_t *component_of_stream(xccl_stream_t *stream, int *mt)
{
    if (stream == NULL || (unsigned)stream->type >= XCCL_STREAM_TYPE_LAST) {
        return NULL;
    }
    *mt = stream_to_mem_type[stream->type];
    return component_of(*mt);
}

/* reference mem_component.c:11-49 */
xccl_status_t xccl_mem_component_init(const char *components_path)
{
    const char *cache_env = getenv("XCCL_MEM_COMPONENT_CACHE_SIZE");
    size_t      cache_size = cache_env ? (size_t)strtoull(cache_env, NULL, 0) : 4096;
    size_t      path_len;
    char       *path, sym[64], *c;
    void       *handle;
    int         mt;

    if (components_path == NULL) {
        return XCCL_ERR_INVALID_PARAM;
    }
    path_len = strlen(components_path) + 64;
    path     = (char *)malloc(path_len);
    if (path == NULL) {
        return XCCL_ERR_NO_MEMORY;
    }

    for (mt = UCS_MEMORY_TYPE_HOST + 1; mt < UCS_MEMORY_TYPE_LAST; mt++) {
        xccl_mem_component_t *mc;

        if (mem_components[mt] != NULL) {
            continue; /* already loaded by an earlier init */
        }
        snprintf(path, path_len, "%s/xccl_%s_mem_component.so", components_path, memory_type_names[mt]);
        handle = dlopen(path, RTLD_LAZY);
        if (handle == NULL) {
            continue;
        }
        snprintf(sym, sizeof(sym), "xccl_%s_mem_component", memory_type_names[mt]);
        for (c = sym; *c; c++) {
            if (*c == '-') {
                *c = '_';
            }
        }
        mc = (xccl_mem_component_t *)dlsym(handle, sym);
        if (mc == NULL) {
            mc = (xccl_mem_component_t *)dlsym(handle, "xccl_cuda_mem_component");
        }
        if (mc == NULL || mc->open() != XCCL_OK) {
            dlclose(handle);
            continue;
        }
        {
            /* the extension announces itself through a symbol of its own,
             * xccl_<name>_mem_component_ext, which points at the object */
            xccl_rocm_mem_component_t **ext;

            strncat(sym, "_ext", sizeof(sym) - strlen(sym) - 1);
            ext = (xccl_rocm_mem_component_t **)dlsym(handle, sym);
            mem_extensions[mt] = (ext != NULL && *ext != NULL && &(*ext)->super == mc &&
                                  (*ext)->ext_version >= 1) ? *ext : NULL;
        }
        mc->dlhandle       = handle;
        mc->cache.size     = cache_size;
        mc->cache.used     = 0;
        mc->cache.buf      = NULL;
        mem_components[mt] = mc;
    }

    free(path);
    return XCCL_OK;
}

/* reference mem_component.c:51-85 */
xccl_status_t xccl_mem_component_alloc(void **ptr, size_t len, ucs_memory_type_t mt)
{
    xccl_mem_component_t *mc;
    xccl_status_t         st;

    if (mt == UCS_MEMORY_TYPE_HOST) {
        *ptr = malloc(len);
        return *ptr ? XCCL_OK : XCCL_ERR_NO_MEMORY;
    }
    mc = component_of(mt);
    if (mc == NULL) {
        return XCCL_ERR_UNSUPPORTED;
    }
    /* One buffer of cache.size bytes stays allocated and is lent to whichever
     * request fits and finds it idle: the k-nomial scratch of small messages
     * then costs no device allocation (allreduce_knomial.c:181-183).  `used`
     * is claimed atomically: collectives may be posted from several threads
     * (XCCL_THREAD_MODE_MULTIPLE), and two of them must never be lent the
     * same buffer. */
    if (mc->cache.size >= len) {
        int idle = 0;
        if (__atomic_compare_exchange_n(&mc->cache.used, &idle, 1, 0, __ATOMIC_ACQ_REL, __ATOMIC_ACQUIRE)) {
            void *buf = __atomic_load_n(&mc->cache.buf, __ATOMIC_ACQUIRE);
            if (buf == NULL) {
                st = mc->mem_alloc(&buf, mc->cache.size);
                if (st != XCCL_OK) {
                    __atomic_store_n(&mc->cache.used, 0, __ATOMIC_RELEASE);
                    return st;
                }
                __atomic_store_n(&mc->cache.buf, buf, __ATOMIC_RELEASE);
            }
            *ptr = buf;
            return XCCL_OK;
        }
    }
    return mc->mem_alloc(ptr, len);
}

/* reference mem_component.c:87-105 */
xccl_status_t xccl_mem_component_free(void *ptr, ucs_memory_type_t mt)
{
    xccl_mem_component_t *mc;

    if (mt == UCS_MEMORY_TYPE_HOST) {
        free(ptr);
        return XCCL_OK;
    }
    mc = component_of(mt);
    if (mc == NULL) {
        return XCCL_ERR_UNSUPPORTED;
    }
    if (ptr != NULL && ptr == __atomic_load_n(&mc->cache.buf, __ATOMIC_ACQUIRE)) {
        __atomic_store_n(&mc->cache.used, 0, __ATOMIC_RELEASE);
        return XCCL_OK;
    }
    return mc->mem_free(ptr);
}

/* reference mem_component.c:107-120 */
xccl_status_t xccl_mem_component_reduce(void *sbuf1, void *sbuf2, void *target, size_t count, xccl_dt_t dtype,
                                        xccl_op_t op, ucs_memory_type_t mt)
{
    xccl_mem_component_t *mc = component_of(mt);

    if (mc == NULL) {
        return XCCL_ERR_UNSUPPORTED; /* includes HOST: no CPU arithmetic here */
    }
    return mc->reduce(sbuf1, sbuf2, target, count, dtype, op);
}

/* reference mem_component.c:122-148 */
xccl_status_t xccl_mem_component_reduce_multi(void *sbuf1, void *sbuf2, void *rbuf, size_t count, size_t size,
                                              size_t stride, xccl_dt_t dtype, xccl_op_t op, ucs_memory_type_t mt)
{
    xccl_mem_component_t *mc;

    if (size == 0) {
        return XCCL_OK;
    }
    mc = component_of(mt);
    if (mc == NULL) {
        return XCCL_ERR_UNSUPPORTED;
    }
    return mc->reduce_multi(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op);
}

/*
 * Stream-ordered forms -- the same entries, argument for argument and rule
 * for rule, that integration/xccl-rocm.patch adds to the reference's
 * src/utils/mem_component.{h,c}:
 *   - *event (if asked for) is NULL whenever the reduction is complete on
 *     return;
 *   - host memory or no component: the blocking dispatcher entry decides;
 *   - a component without the extension: the blocking entry when the call
 *     names no stream, XCCL_ERR_NOT_IMPLEMENTED when it does;
 *   - an empty reduction is XCCL_OK;
 *   - an empty event pool (XCCL_ERR_NO_RESOURCE from the component, nothing
 *     enqueued): the blocking entry when the call names no stream, the error
 *     when it does.
 */
xccl_status_t xccl_mem_component_reduce_nb(void *sbuf1, void *sbuf2, void *target, size_t count, xccl_dt_t dtype,
                                           xccl_op_t op, ucs_memory_type_t mt, xccl_stream_t *stream,
                                           xccl_mc_event_t **event)
{
    xccl_mem_component_t      *mc  = component_of(mt);
    xccl_rocm_mem_component_t *ext = extension_of(mt);
    xccl_status_t              st;

    if (event != NULL) {
        *event = NULL;
    }
    if (mc == NULL || (ext == NULL && stream == NULL)) {
        return xccl_mem_component_reduce(sbuf1, sbuf2, target, count, dtype, op, mt);
    }
    if (ext == NULL) {
        return XCCL_ERR_NOT_IMPLEMENTED;
    }
    if (count == 0) {
        return XCCL_OK;
    }
    st = ext->reduce_nb(sbuf1, sbuf2, target, count, dtype, op, stream, event);
    if (st == XCCL_ERR_NO_RESOURCE && stream == NULL) {
        return mc->reduce(sbuf1, sbuf2, target, count, dtype, op);
    }
    if (st == XCCL_OK && event != NULL) {
        (*event)->mem_type = mt;
    }
    return st;
}

xccl_status_t xccl_mem_component_reduce_multi_nb(void *sbuf1, void *sbuf2, void *rbuf, size_t count, size_t size,
                                                 size_t stride, xccl_dt_t dtype, xccl_op_t op, ucs_memory_type_t mt,
                                                 xccl_stream_t *stream, xccl_mc_event_t **event)
{
    xccl_mem_component_t      *mc  = component_of(mt);
    xccl_rocm_mem_component_t *ext = extension_of(mt);
    xccl_status_t              st;

    if (event != NULL) {
        *event = NULL;
    }
    if (mc == NULL || (ext == NULL && stream == NULL)) {
        return xccl_mem_component_reduce_multi(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, mt);
    }
    if (ext == NULL) {
        return XCCL_ERR_NOT_IMPLEMENTED;
    }
    if (size == 0) {
        return XCCL_OK;
    }
    st = ext->reduce_multi_nb(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, stream, event);
    if (st == XCCL_ERR_NO_RESOURCE && stream == NULL) {
        return mc->reduce_multi(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op);
    }
    if (st == XCCL_OK && event != NULL) {
        (*event)->mem_type = mt;
    }
    return st;
}

/* reference mem_component.c:150-174: the first component, in memory-type
 * order, that recognises the pointer decides; nobody does -> HOST. */
xccl_status_t xccl_mem_component_type(void *ptr, ucs_memory_type_t *mem_type)
{
    int mt;

    *mem_type = UCS_MEMORY_TYPE_LAST;
    for (mt = UCS_MEMORY_TYPE_HOST + 1; mt < UCS_MEMORY_TYPE_LAST; mt++) {
        if (mem_components[mt] == NULL) {
            continue;
        }
        if (mem_components[mt]->mem_type(ptr, mem_type) == XCCL_OK && *mem_type != UCS_MEMORY_TYPE_LAST) {
            return XCCL_OK;
        }
    }
    *mem_type = UCS_MEMORY_TYPE_HOST;
    return XCCL_OK;
}

/* reference mem_component.c:180-195 */
xccl_status_t xccl_mem_component_memcpy_async(void *sbuf, void *dbuf, size_t size, xccl_stream_t *stream)
{
    xccl_mem_component_t *mc;
    int                   mt;

    if (size == 0) {
        return XCCL_OK;
    }
    mc = component_of_stream(stream, &mt);
    if (mc == NULL) {
        return XCCL_ERR_UNSUPPORTED;
    }
    return mc->memcpy_async(sbuf, dbuf, size, stream);
}

/* reference mem_component.c:197-213 */
xccl_status_t xccl_mem_component_start_acitivity(xccl_stream_t *stream, xccl_mem_component_stream_request_t **req)
{
    xccl_mem_component_t *mc;
    xccl_status_t         st;
    int                   mt;

    mc = component_of_stream(stream, &mt);
    if (mc == NULL) {
        return XCCL_ERR_UNSUPPORTED;
    }
    st = mc->start_stream_activity(stream, req);
    if (st == XCCL_OK) {
        (*req)->mem_type = (ucs_memory_type_t)mt;
    }
    return st;
}

/* reference mem_component.c:215-229 */
xccl_status_t xccl_mem_component_finish_acitivity(xccl_mem_component_stream_request_t *req)
{
    xccl_mem_component_t *mc = req ? component_of(req->mem_type) : NULL;

    if (mc == NULL) {
        return XCCL_ERR_UNSUPPORTED;
    }
    return mc->finish_stream_activity(req);
}

/* reference mem_component.c:231-247 */
xccl_status_t xccl_mc_event_record(xccl_stream_t *stream, xccl_mc_event_t **event)
{
    xccl_mem_component_t *mc;
    xccl_status_t         st;
    int                   mt;

    mc = component_of_stream(stream, &mt);
    if (mc == NULL) {
        return XCCL_ERR_UNSUPPORTED;
    }
    st = mc->event_record(stream, event);
    if (st == XCCL_OK) {
        (*event)->mem_type = (ucs_memory_type_t)mt;
    }
    return st;
}

/* reference mem_component.c:249-252 */
xccl_status_t xccl_mc_event_query(xccl_mc_event_t *event)
{
    xccl_mem_component_t *mc = event ? component_of(event->mem_type) : NULL;

    return mc ? mc->event_query(event) : XCCL_ERR_UNSUPPORTED;
}

/* reference mem_component.c:254-257 */
xccl_status_t xccl_mc_event_free(xccl_mc_event_t *event)
{
    xccl_mem_component_t *mc = event ? component_of(event->mem_type) : NULL;

    return mc ? mc->event_free(event) : XCCL_ERR_UNSUPPORTED;
}

xccl_status_t xccl_mc_event_wait(xccl_mc_event_t *event)
{
    xccl_rocm_mem_component_t *ext;

    if (event == NULL || component_of(event->mem_type) == NULL) {
        return XCCL_ERR_UNSUPPORTED;
    }
    ext = extension_of(event->mem_type);
    return ext ? ext->event_wait(event) : XCCL_ERR_NOT_IMPLEMENTED;
}

/* reference mem_component.c:259-272 */
void xccl_mem_component_free_cache(void)
{
    int mt;

    for (mt = UCS_MEMORY_TYPE_HOST + 1; mt < UCS_MEMORY_TYPE_LAST; mt++) {
        xccl_mem_component_t *mc = mem_components[mt];
        if (mc == NULL) {
            continue;
        }
        if (mc->cache.buf != NULL && !__atomic_load_n(&mc->cache.used, __ATOMIC_ACQUIRE)) {
            mc->mem_free(mc->cache.buf);
            mc->cache.buf = NULL;
        }
        mc->close();
    }
}

/* reference mem_component.c:274-283 */
void xccl_mem_component_finalize(void)
{
    int mt;

    for (mt = UCS_MEMORY_TYPE_HOST + 1; mt < UCS_MEMORY_TYPE_LAST; mt++) {
        if (mem_components[mt] != NULL) {
            void *handle       = mem_components[mt]->dlhandle;
            mem_components[mt] = NULL;
            mem_extensions[mt] = NULL;
            dlclose(handle);
        }
    }
}

xccl_mem_component_t *xccl_mem_component_get(ucs_memory_type_t mem_type)
{
    return component_of(mem_type);
}
