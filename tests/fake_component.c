/* A host-memory stand-in component for dispatcher tests: exports the one data
 * symbol the reference loader looks up (src/utils/mem_component.c:30), counts
 * calls, and serves "device" memory from malloc.  With -DFAKE_EXT_SYMBOL=<name>
 * the object carries the stream-ordered extension and <name> points at it;
 * fake_set_nb_status() chooses what its reduce_nb / reduce_multi_nb return.
 * Not a product file. */
#include <stdlib.h>
#include <string.h>

#include "xccl_rocm_mem_component.h"

int fake_calls[16];
static int fake_open_status = 0;
enum { C_OPEN, C_ALLOC, C_FREE, C_TYPE, C_REDUCE, C_REDUCE_MULTI, C_MEMCPY, C_EV_REC, C_EV_QUERY, C_EV_FREE,
       C_START, C_FINISH, C_CLOSE, C_REDUCE_NB, C_REDUCE_MULTI_NB };

/* several threads call at once in the stress tests */
#define COUNT(_i) __atomic_fetch_add(&fake_calls[_i], 1, __ATOMIC_RELAXED)

size_t fake_last_args[8];
static char fake_arena[1 << 16];
static xccl_mc_event_t fake_event;
static xccl_mem_component_stream_request_t fake_req;

static xccl_status_t f_open(void) { COUNT(C_OPEN); return (xccl_status_t)fake_open_status; }
static xccl_status_t f_alloc(void **p, size_t len) { COUNT(C_ALLOC); *p = malloc(len ? len : 1); return XCCL_OK; }
static xccl_status_t f_free(void *p) { COUNT(C_FREE); free(p); return XCCL_OK; }
static xccl_status_t f_type(void *p, ucs_memory_type_t *mt)
{
    COUNT(C_TYPE);
    if ((char *)p >= fake_arena && (char *)p < fake_arena + sizeof(fake_arena)) {
        *mt = FAKE_MEMTYPE;
        return XCCL_OK;
    }
    return XCCL_ERR_UNSUPPORTED;
}
static xccl_status_t f_reduce(void *a, void *b, void *t, size_t n, xccl_dt_t dt, xccl_op_t op)
{
    COUNT(C_REDUCE);
    fake_last_args[0] = (size_t)a; fake_last_args[1] = (size_t)b; fake_last_args[2] = (size_t)t;
    fake_last_args[3] = n; fake_last_args[4] = (size_t)dt; fake_last_args[5] = (size_t)op;
    return XCCL_OK;
}
static xccl_status_t f_reduce_multi(void *a, void *b, void *t, size_t cnt, size_t size, size_t stride, xccl_dt_t dt,
                                    xccl_op_t op)
{
    COUNT(C_REDUCE_MULTI);
    fake_last_args[0] = (size_t)a; fake_last_args[1] = (size_t)b; fake_last_args[2] = (size_t)t;
    fake_last_args[3] = cnt; fake_last_args[4] = size; fake_last_args[5] = stride;
    fake_last_args[6] = (size_t)dt; fake_last_args[7] = (size_t)op;
    return XCCL_OK;
}
static xccl_status_t f_memcpy(void *s, void *d, size_t n, xccl_stream_t *st) { (void)st; COUNT(C_MEMCPY); memcpy(d, s, n); return XCCL_OK; }
static xccl_status_t f_ev_rec(xccl_stream_t *s, xccl_mc_event_t **e) { (void)s; COUNT(C_EV_REC); *e = &fake_event; return XCCL_OK; }
static xccl_status_t f_ev_query(xccl_mc_event_t *e) { (void)e; COUNT(C_EV_QUERY); return XCCL_INPROGRESS; }
static xccl_status_t f_ev_free(xccl_mc_event_t *e) { (void)e; COUNT(C_EV_FREE); return XCCL_OK; }
static xccl_status_t f_start(xccl_stream_t *s, xccl_mem_component_stream_request_t **r) { (void)s; COUNT(C_START); *r = &fake_req; return XCCL_OK; }
static xccl_status_t f_finish(xccl_mem_component_stream_request_t *r) { (void)r; COUNT(C_FINISH); return XCCL_OK; }
static void f_close(void) { COUNT(C_CLOSE); }

void *fake_arena_ptr(void) { return fake_arena; }
void fake_set_open_status(int s) { fake_open_status = s; }

#define FAKE_VTABLE                                                                                      \
    {                                                                                                    \
        f_open, f_alloc, f_free, f_type, f_reduce, f_reduce_multi, f_memcpy, f_ev_rec, f_ev_query,      \
        f_ev_free, f_start, f_finish, f_close, 0, {0, 0, 0}                                              \
    }

#ifdef FAKE_EXT_SYMBOL
static int fake_nb_status = 0;
void      *fake_last_stream;
void fake_set_nb_status(int s) { fake_nb_status = s; }

static xccl_status_t nb_result(xccl_stream_t *stream, xccl_mc_event_t **event)
{
    fake_last_stream = stream;
    if (fake_nb_status == XCCL_OK && event != NULL) {
        *event = &fake_event;
    }
    return (xccl_status_t)fake_nb_status;
}
static xccl_status_t f_reduce_nb(void *a, void *b, void *t, size_t n, xccl_dt_t dt, xccl_op_t op,
                                 xccl_stream_t *stream, xccl_mc_event_t **event)
{
    (void)a; (void)b; (void)t; (void)n; (void)dt; (void)op;
    COUNT(C_REDUCE_NB);
    return nb_result(stream, event);
}
static xccl_status_t f_reduce_multi_nb(void *a, void *b, void *t, size_t cnt, size_t size, size_t stride,
                                       xccl_dt_t dt, xccl_op_t op, xccl_stream_t *stream, xccl_mc_event_t **event)
{
    (void)a; (void)b; (void)t; (void)cnt; (void)size; (void)stride; (void)dt; (void)op;
    COUNT(C_REDUCE_MULTI_NB);
    return nb_result(stream, event);
}
static xccl_status_t f_ev_wait(xccl_mc_event_t *e) { (void)e; return XCCL_OK; }
static xccl_status_t f_get_stream(void **s) { *s = NULL; return XCCL_OK; }

xccl_rocm_mem_component_t FAKE_SYMBOL = {FAKE_VTABLE, 1, f_reduce_nb, f_reduce_multi_nb, f_ev_wait, f_get_stream};
xccl_rocm_mem_component_t *const FAKE_EXT_SYMBOL = &FAKE_SYMBOL;
#else
xccl_mem_component_t FAKE_SYMBOL = FAKE_VTABLE;
#endif
