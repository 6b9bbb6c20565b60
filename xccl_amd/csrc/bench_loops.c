/*
 * bench_loops.c -- timing loops for the small-message latency sweep, in C so
 * that the per-call figure holds no interpreter overhead.  Part of
 * libxccl_rocm_benchkit.so (bench and tests only; not loaded by the
 * component).  The component is reached through the pointer the caller
 * passes, i.e. through the same exported object libxccl would use.
 */
#include "xccl_rocm_kernels.h"
#include "xccl_rocm_mem_component.h"

#include <hip/hip_runtime_api.h>
#include <time.h>

static inline uint64_t now_ns(void)
{
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (uint64_t)ts.tv_sec * 1000000000ull + (uint64_t)ts.tv_nsec;
}

typedef xccl_status_t (*graph_fn_t)(void *, void *, void *, size_t, size_t, size_t, xccl_dt_t, xccl_op_t, void *);

/*
 * Runs `iters` back-to-back reduce_multi calls and stores each call's
 * host-observed duration (entry to completion seen by the host) in ns_out.
 *   mode 0: the synchronous vtable entry (launch + stream synchronize inside)
 *   mode 1: reduce_multi_nb on the component stream + event_query polling
 *   mode 2: `graph_fn` (xccl_rocm_reduce_multi_graph) + hipStreamSynchronize
 *   mode 3: reduce_multi_nb without event + hipStreamSynchronize
 *   mode 4: reduce_multi_nb + event; only the call itself is timed (the host's
 *           cost of issuing one reduction), the wait that follows is not
 * Returns the first non-OK status, or XCCL_OK.
 */
xccl_status_t xccl_rocm_bench_latency(xccl_rocm_mem_component_t *mc, graph_fn_t graph_fn, int mode, void *sbuf1,
                                      void *sbuf2, void *rbuf, size_t count, size_t size, size_t stride,
                                      xccl_dt_t dtype, xccl_op_t op, size_t iters, uint64_t *ns_out)
{
    void         *stream = NULL;
    xccl_status_t st     = mc->get_stream(&stream);
    size_t        i;

    if (st != XCCL_OK) {
        return st;
    }
    for (i = 0; i < iters; i++) {
        const uint64_t t0 = now_ns();
        if (mode == 0) {
            st = mc->super.reduce_multi(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op);
        } else if (mode == 1) {
            xccl_mc_event_t *ev = NULL;
            st = mc->reduce_multi_nb(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, NULL, &ev);
            if (st == XCCL_OK) {
                while ((st = mc->super.event_query(ev)) == XCCL_INPROGRESS) {
                }
                mc->super.event_free(ev);
            }
        } else if (mode == 2) {
            st = graph_fn(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, stream);
            if (st == XCCL_OK && hipStreamSynchronize((hipStream_t)stream) != hipSuccess) {
                st = XCCL_ERR_NO_MESSAGE;
            }
        } else if (mode == 4) {
            xccl_mc_event_t *ev = NULL;
            st        = mc->reduce_multi_nb(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, NULL, &ev);
            ns_out[i] = now_ns() - t0;
            if (st == XCCL_OK) {
                st = mc->event_wait(ev);
                mc->super.event_free(ev);
            }
            if (st != XCCL_OK) {
                return st;
            }
            continue;
        } else {
            st = mc->reduce_multi_nb(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, NULL, NULL);
            if (st == XCCL_OK && hipStreamSynchronize((hipStream_t)stream) != hipSuccess) {
                st = XCCL_ERR_NO_MESSAGE;
            }
        }
        ns_out[i] = now_ns() - t0;
        if (st != XCCL_OK) {
            return st;
        }
    }
    return XCCL_OK;
}

/*
 * Enqueues `iters` stream-ordered reduce_multi calls back to back on the
 * component stream, each bracketed by its own pair of timing events, waits
 * once, and stores each launch's device-side duration in ms_out.  `ev` holds
 * 2*iters timing-enabled hipEvent_t created by the caller.
 */
xccl_status_t xccl_rocm_bench_kernel_times(xccl_rocm_mem_component_t *mc, void *sbuf1, void *sbuf2, void *rbuf,
                                           size_t count, size_t size, size_t stride, xccl_dt_t dtype, xccl_op_t op,
                                           size_t iters, void **ev, float *ms_out)
{
    void         *stream = NULL;
    xccl_status_t st     = mc->get_stream(&stream);
    size_t        i;

    if (st != XCCL_OK) {
        return st;
    }
    for (i = 0; i < iters; i++) {
        if (hipEventRecord((hipEvent_t)ev[2 * i], (hipStream_t)stream) != hipSuccess) {
            return XCCL_ERR_NO_MESSAGE;
        }
        st = mc->reduce_multi_nb(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, NULL, NULL);
        if (st != XCCL_OK) {
            return st;
        }
        if (hipEventRecord((hipEvent_t)ev[2 * i + 1], (hipStream_t)stream) != hipSuccess) {
            return XCCL_ERR_NO_MESSAGE;
        }
    }
    if (hipStreamSynchronize((hipStream_t)stream) != hipSuccess) {
        return XCCL_ERR_NO_MESSAGE;
    }
    for (i = 0; i < iters; i++) {
        if (hipEventElapsedTime(&ms_out[i], (hipEvent_t)ev[2 * i], (hipEvent_t)ev[2 * i + 1]) != hipSuccess) {
            return XCCL_ERR_NO_MESSAGE;
        }
    }
    return XCCL_OK;
}

/*
 * Times `iters` mem_type probes of `ptr` (the query libxccl issues at least
 * twice per collective, reference src/utils/mem_component.c:150-174) and
 * stores each call's duration in ns_out; *mt_out receives the last answer
 * (UCS_MEMORY_TYPE_LAST if the component did not recognise the pointer).
 */
xccl_status_t xccl_rocm_bench_mem_type(xccl_rocm_mem_component_t *mc, void *ptr, size_t iters, uint64_t *ns_out,
                                       int *mt_out)
{
    ucs_memory_type_t mt = UCS_MEMORY_TYPE_LAST;
    size_t            i;

    for (i = 0; i < iters; i++) {
        const uint64_t t0 = now_ns();
        if (mc->super.mem_type(ptr, &mt) != XCCL_OK) {
            mt = UCS_MEMORY_TYPE_LAST;
        }
        ns_out[i] = now_ns() - t0;
    }
    *mt_out = (int)mt;
    return XCCL_OK;
}

/*
 * Times `iters` mem_alloc(len) + mem_free pairs through the component's
 * vtable -- what one collective pays for its scratch buffer (reference
 * allreduce_knomial.c:181-183 and xccl_ucx_allreduce_knomial's completion) --
 * and stores each pair's duration in ns_out.
 */
xccl_status_t xccl_rocm_bench_alloc_free(xccl_rocm_mem_component_t *mc, size_t len, size_t iters, uint64_t *ns_out)
{
    size_t i;

    for (i = 0; i < iters; i++) {
        void          *p  = NULL;
        const uint64_t t0 = now_ns();
        xccl_status_t  st = mc->super.mem_alloc(&p, len);
        if (st != XCCL_OK) {
            return st;
        }
        st = mc->super.mem_free(p);
        ns_out[i] = now_ns() - t0;
        if (st != XCCL_OK) {
            return st;
        }
    }
    return XCCL_OK;
}

/*
 * One pair of timing events around `iters` stream-ordered reduce_multi calls
 * enqueued back to back on the component stream: *ms_out is the whole
 * region's device time, so region / iters is the average launch duration
 * without a per-launch event's own cost (about 5 us per pair on this part).
 */
xccl_status_t xccl_rocm_bench_region_time(xccl_rocm_mem_component_t *mc, void *sbuf1, void *sbuf2, void *rbuf,
                                          size_t count, size_t size, size_t stride, xccl_dt_t dtype, xccl_op_t op,
                                          size_t iters, void *ev_begin, void *ev_end, float *ms_out)
{
    void         *stream = NULL;
    xccl_status_t st     = mc->get_stream(&stream);
    size_t        i;

    if (st != XCCL_OK) {
        return st;
    }
    if (hipEventRecord((hipEvent_t)ev_begin, (hipStream_t)stream) != hipSuccess) {
        return XCCL_ERR_NO_MESSAGE;
    }
    for (i = 0; i < iters; i++) {
        st = mc->reduce_multi_nb(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, NULL, NULL);
        if (st != XCCL_OK) {
            return st;
        }
    }
    if (hipEventRecord((hipEvent_t)ev_end, (hipStream_t)stream) != hipSuccess ||
        hipStreamSynchronize((hipStream_t)stream) != hipSuccess ||
        hipEventElapsedTime(ms_out, (hipEvent_t)ev_begin, (hipEvent_t)ev_end) != hipSuccess) {
        return XCCL_ERR_NO_MESSAGE;
    }
    return XCCL_OK;
}

/*
 * xccl_rocm_bench_region_time with the destination cycling through
 * `rot_count` vectors `rot_pitch` bytes apart (launch i writes rbuf +
 * (i % rot_count) * rot_pitch): a destination that is rewritten launch after
 * launch partly stays in the memory-side cache, a rotating one does not.
 */
xccl_status_t xccl_rocm_bench_region_time_rot(xccl_rocm_mem_component_t *mc, void *sbuf1, void *sbuf2, void *rbuf,
                                              size_t rot_count, size_t rot_pitch, size_t count, size_t size,
                                              size_t stride, xccl_dt_t dtype, xccl_op_t op, size_t iters,
                                              void *ev_begin, void *ev_end, float *ms_out)
{
    void         *stream = NULL;
    xccl_status_t st     = mc->get_stream(&stream);
    size_t        i;

    if (st != XCCL_OK) {
        return st;
    }
    if (rot_count == 0) {
        return XCCL_ERR_INVALID_PARAM;
    }
    if (hipEventRecord((hipEvent_t)ev_begin, (hipStream_t)stream) != hipSuccess) {
        return XCCL_ERR_NO_MESSAGE;
    }
    for (i = 0; i < iters; i++) {
        st = mc->reduce_multi_nb(sbuf1, sbuf2, (char *)rbuf + (i % rot_count) * rot_pitch, count, size, stride, dtype,
                                 op, NULL, NULL);
        if (st != XCCL_OK) {
            return st;
        }
    }
    if (hipEventRecord((hipEvent_t)ev_end, (hipStream_t)stream) != hipSuccess ||
        hipStreamSynchronize((hipStream_t)stream) != hipSuccess ||
        hipEventElapsedTime(ms_out, (hipEvent_t)ev_begin, (hipEvent_t)ev_end) != hipSuccess) {
        return XCCL_ERR_NO_MESSAGE;
    }
    return XCCL_OK;
}

/*
 * `threads` host threads (at most 16) call the blocking reduce_multi entry at
 * the same time, `iters` times each, every thread on operands of its own
 * (thread t uses sbuf1 + t * thread_pitch and so on); ns_out receives
 * threads * iters per-call durations, thread after thread.  What a
 * XCCL_THREAD_MODE_MULTIPLE application sees (reference test/test_mt.c).
 */
#include <pthread.h>

typedef struct {
    xccl_rocm_mem_component_t *mc;
    char                      *s1, *s2, *out;
    size_t                     count, size, stride, iters;
    xccl_dt_t                  dtype;
    xccl_op_t                  op;
    uint64_t                  *ns;
    xccl_status_t              st;
} mt_arg_t;

static void *mt_worker(void *p)
{
    mt_arg_t *a = (mt_arg_t *)p;
    size_t    i;

    for (i = 0; i < a->iters && a->st == XCCL_OK; i++) {
        const uint64_t t0 = now_ns();
        a->st    = a->mc->super.reduce_multi(a->s1, a->s2, a->out, a->count, a->size, a->stride, a->dtype, a->op);
        a->ns[i] = now_ns() - t0;
    }
    return NULL;
}

xccl_status_t xccl_rocm_bench_latency_mt(xccl_rocm_mem_component_t *mc, int threads, size_t thread_pitch, void *sbuf1,
                                         void *sbuf2, void *rbuf, size_t count, size_t size, size_t stride,
                                         xccl_dt_t dtype, xccl_op_t op, size_t iters, uint64_t *ns_out)
{
    pthread_t th[16];
    mt_arg_t  arg[16];
    int       t;

    if (threads < 1 || threads > 16) {
        return XCCL_ERR_INVALID_PARAM;
    }
    for (t = 0; t < threads; t++) {
        arg[t] = (mt_arg_t){mc, (char *)sbuf1 + t * thread_pitch, (char *)sbuf2 + t * thread_pitch,
                            (char *)rbuf + t * thread_pitch, count, size, stride, iters, dtype, op,
                            ns_out + (size_t)t * iters, XCCL_OK};
        if (pthread_create(&th[t], NULL, mt_worker, &arg[t]) != 0) {
            threads = t;
            break;
        }
    }
    for (t = 0; t < threads; t++) {
        pthread_join(th[t], NULL);
    }
    for (t = 0; t < threads; t++) {
        if (arg[t].st != XCCL_OK) {
            return arg[t].st;
        }
    }
    return XCCL_OK;
}

/*
 * Times `iters` rounds of memcpy_async(src -> dst, len) on `xs` followed by
 * event_record and event_query polling until done -- one message of the
 * loopback transport, or one step of the mpod team library's alltoall
 * (reference src/team_lib/mpod/xccl_mpod_alltoall.c:41-163 uses the
 * same three entries).
 */
xccl_status_t xccl_rocm_bench_memcpy(xccl_rocm_mem_component_t *mc, xccl_stream_t *xs, void *src, void *dst, size_t len,
                                     size_t iters, uint64_t *ns_out)
{
    size_t i;

    for (i = 0; i < iters; i++) {
        xccl_mc_event_t *ev = NULL;
        const uint64_t   t0 = now_ns();
        xccl_status_t    st = mc->super.memcpy_async(src, dst, len, xs);
        if (st != XCCL_OK) {
            return st;
        }
        st = mc->super.event_record(xs, &ev);
        if (st != XCCL_OK) {
            return st;
        }
        while ((st = mc->super.event_query(ev)) == XCCL_INPROGRESS) {
        }
        mc->super.event_free(ev);
        ns_out[i] = now_ns() - t0;
        if (st != XCCL_OK) {
            return st;
        }
    }
    return XCCL_OK;
}

/*
 * Where the time of a one-node graph launch goes.  Each of `iters` rounds
 * issues one reduction through `graph_fn` (xccl_rocm_reduce_multi_graph_flagged)
 * with a completion word, then polls the word's host view until the kernel has
 * written it.  ns_out receives 6 values per round: planning, lock + slot
 * search, patching the node, hipGraphLaunch, launch-returned-to-completion-seen,
 * and the whole round.  The counters and the word are allocated here (bench
 * code; the component's own come from its event pool).
 */
typedef xccl_status_t (*graph_flagged_fn_t)(void *, void *, void *, size_t, size_t, size_t, xccl_dt_t, xccl_op_t,
                                            void *, uint32_t *, uint32_t *, uint32_t, int *, uint64_t *);

xccl_status_t xccl_rocm_bench_graph_parts(xccl_rocm_mem_component_t *mc, graph_flagged_fn_t graph_fn, void *sbuf1,
                                          void *sbuf2, void *rbuf, size_t count, size_t size, size_t stride,
                                          xccl_dt_t dtype, xccl_op_t op, size_t iters, uint64_t *ns_out)
{
    void              *stream = NULL;
    uint32_t          *counters = NULL, *dev_flag = NULL;
    volatile uint32_t *flag = NULL;
    xccl_status_t      st = mc->get_stream(&stream);
    size_t             i;

    if (st != XCCL_OK) {
        return st;
    }
    if (hipMalloc((void **)&counters, XCCL_ROCM_DONE_COUNT_BYTES) != hipSuccess ||
        hipMemset(counters, 0, XCCL_ROCM_DONE_COUNT_BYTES) != hipSuccess ||
        hipHostMalloc((void **)&flag, 64, hipHostMallocMapped) != hipSuccess ||
        hipHostGetDevicePointer((void **)&dev_flag, (void *)flag, 0) != hipSuccess) {
        return XCCL_ERR_NO_MESSAGE;
    }
    *flag = 0;
    for (i = 0; i < iters && st == XCCL_OK; i++) {
        uint64_t       parts[4] = {0, 0, 0, 0};
        int            flagged  = 0;
        const uint64_t t0       = now_ns();
        uint64_t       t1;
        st = graph_fn(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, stream, counters, dev_flag, (uint32_t)(i + 1),
                      &flagged, parts);
        t1 = now_ns();
        if (st != XCCL_OK) {
            break;
        }
        if (flagged) {
            while (__atomic_load_n(flag, __ATOMIC_ACQUIRE) != (uint32_t)(i + 1)) {
            }
        } else if (hipStreamSynchronize((hipStream_t)stream) != hipSuccess) {
            st = XCCL_ERR_NO_MESSAGE;
        }
        ns_out[6 * i + 0] = parts[0];
        ns_out[6 * i + 1] = parts[1];
        ns_out[6 * i + 2] = parts[2];
        ns_out[6 * i + 3] = parts[3];
        ns_out[6 * i + 4] = now_ns() - t1;
        ns_out[6 * i + 5] = now_ns() - t0;
    }
    (void)hipStreamSynchronize((hipStream_t)stream);
    (void)hipFree(counters);
    (void)hipHostFree((void *)flag);
    return st;
}
