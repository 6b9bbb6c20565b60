/*
 * mc_rocm.c -- the ROCm memory component of XCCL: the object that
 * xccl_rocm_mem_component.so exports and libxccl's mem-component dispatcher
 * calls through (vtable: reference src/utils/mem_component.h:28-49).
 *
 * It stands where the reference's CUDA component stands
 * (src/utils/cuda/cuda_mem_component.c) and keeps that component's contract:
 * per-process singletons, resources created on first use (open() runs inside
 * libxccl's ELF constructor, before the application picked a device --
 * cuda_mem_component.c:18-32), synchronous reduce / reduce_multi, pooled
 * events and stream requests, XCCL_ERR_NO_MESSAGE for runtime failures,
 * XCCL_ERR_NO_RESOURCE for an empty pool, XCCL_ERR_UNSUPPORTED for a
 * (dtype, op) without a kernel.  It differs where the reference is unsafe or
 * slow:
 *   - resources are kept per device ordinal, and pool slots are claimed with
 *     atomics (the ucx team library advertises XCCL_THREAD_MODE_MULTIPLE,
 *     src/team_lib/ucx/xccl_ucx_lib.c:631-632);
 *   - events are created once (the reference re-creates one on every record,
 *     cuda_mem_component.c:220, and leaks the old one);
 *   - calling threads are spread over up to four reduction streams, and a
 *     stream gate goes into the user's stream, not in front of reductions;
 *   - freed device blocks are cached for the next mem_alloc (mc_pool.h);
 *   - small launches report completion through a host-mapped word the kernel
 *     writes itself, which the host sees sooner than the queue's signal;
 *   - blocking reductions that complete through that word are launched on a
 *     dispatch queue of the component's own (xccl_rocm_reduce_multi_direct),
 *     not through hipLaunchKernel on a stream;
 *   - the vtable is extended with stream-ordered reductions whose completion
 *     is an event (see include/xccl_rocm_mem_component.h).
 *
 * Plain C on the HIP runtime's C API; the kernels are reached through
 * include/xccl_rocm_kernels.h only.
 */
#include "xccl_rocm_kernels.h"
#include "xccl_rocm_mem_component.h"
#include "xccl_rocm_mem_pool.h"
#include "mc_pool.h"

#include <hip/hip_runtime_api.h>
#include <pthread.h>
#include <stdatomic.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define MC_MAX_DEVICES 64

/* Reduction streams per device.  Every calling thread sticks to one of them
 * (assigned round-robin on its first call), so that blocking calls from
 * several threads (XCCL_THREAD_MODE_MULTIPLE) do not queue up behind each
 * other's kernels; 4 = the hardware queues a process gets by default. */
#define MC_NUM_STREAMS 4

/* Synchronous reductions of at most this many bytes per vector are launched
 * through the graph path (XCCL_MC_ROCM_GRAPH_MAX_BYTES overrides; 0 = never). */
#define MC_DEFAULT_GRAPH_MAX_BYTES 0

/* Upper bound on how long a stream gate keeps a user stream blocked when
 * finish_stream_activity is never called (XCCL_MC_ROCM_GATE_TIMEOUT_MS). */
#define MC_DEFAULT_GATE_TIMEOUT_MS 30000

/* Bytes of freed device blocks mem_free may keep for the next mem_alloc
 * (XCCL_MC_ROCM_POOL_MAX_BYTES; 0 = keep none).  Sized for a part with 288 GB. */
#define MC_DEFAULT_POOL_MAX_BYTES ((size_t)8 << 30)

/* pool slot states (`is_free` keeps the reference's member name) */
enum { MC_SLOT_BUSY = 0, MC_SLOT_FREE = 1, MC_SLOT_DRAINING = 2 };

/* An event completes either through its HIP event, or -- when it stands for a
 * small reduction launch -- through a host-mapped word the kernel itself
 * stores a sequence number to (cheaper to observe than the queue's completion
 * signal by ~4 us on this part). */
typedef struct mc_rocm_event {
    xccl_mc_event_t    super;
    atomic_int         is_free;
    hipEvent_t         hip_event;
    int                flagged;   /* n > 0: done when the first n words at flag all equal expect; -1: when `signal` reads 0 */
    uint64_t           signal;    /* completion signal of the own dispatch queue, created when first needed (0: none yet) */
    void              *kernarg;   /* kernel-argument block for launches on the own dispatch queue (pinned host memory) */
    uint32_t           expect;    /* last sequence number handed to a kernel */
    volatile uint32_t *flag;      /* host view of the completion word */
    uint32_t          *dev_flag;  /* device view of the same word */
    uint32_t          *dev_count; /* arrival counters of the launch's workgroups */
    hipStream_t        stream;    /* where the work was enqueued */
    int                direct;    /* 1: launched on the component's own dispatch queue, not on `stream` */
    int                slot;      /* reduction stream the launch went to, -1: a user's stream or the own queue */
    unsigned           stream_seq; /* its number among the launches of that reduction stream */
    struct mc_rocm_device *dev;
    unsigned           polls;
} mc_rocm_event_t;

/* Spin-wait hint: keeps a polling hardware thread from starving its sibling. */
#if defined(__x86_64__) || defined(__i386__)
#define MC_CPU_RELAX() __builtin_ia32_pause()
#elif defined(__aarch64__)
#define MC_CPU_RELAX() __asm__ __volatile__("yield")
#else
#define MC_CPU_RELAX() ((void)0)
#endif

/* uint32 words per event, one 64-byte line: a launch of a handful of workgroups
 * reports on one word per workgroup (xccl_rocm_reduce_multi_slots), every
 * other on the first */
#define MC_FLAG_STRIDE XCCL_ROCM_FLAG_WORDS

typedef struct mc_rocm_stream_request {
    xccl_mem_component_stream_request_t super;
    atomic_int                          is_free;
    int                                *flag;     /* host view of the gate word */
    int                                *dev_flag; /* device view of the same word */
    hipEvent_t                          hip_event;
} mc_rocm_stream_request_t;

typedef struct mc_rocm_device {
    atomic_int               ready; /* 0 = untouched, 1 = usable */
    hipStream_t              stream[MC_NUM_STREAMS]; /* reductions: one per calling thread, round-robin */
    int                     *gate_words;  /* pinned, mapped */
    uint32_t                *flag_words; /* pinned, mapped: completion words of the events */
    uint32_t                *arrival_counts; /* device */
    char                    *kernargs;       /* XCCL_ROCM_KERNARG_BYTES per event: device memory the host can write, else pinned */
    int                      kernargs_pinned; /* 1: ours to free */
    /* Launches put on each reduction stream, and the highest of them known to be complete (the stream runs
     * them in order).  While the two differ, the stream may hold work nobody has waited for, and a call of that
     * slot stays on the stream, behind it, instead of taking the component's own dispatch queue. */
    atomic_uint              stream_issued[MC_NUM_STREAMS];
    atomic_uint              stream_synced[MC_NUM_STREAMS];
    mc_rocm_event_t          events[XCCL_ROCM_MC_NUM_EVENTS];
    mc_rocm_stream_request_t requests[XCCL_ROCM_MC_NUM_STREAM_REQUESTS];
} mc_rocm_device_t;

static mc_rocm_device_t mc_devices[MC_MAX_DEVICES];
static pthread_mutex_t  mc_init_lock = PTHREAD_MUTEX_INITIALIZER;
static size_t           mc_graph_max_bytes;
static int              mc_num_streams = MC_NUM_STREAMS; /* XCCL_MC_ROCM_THREAD_STREAMS, 1 .. MC_NUM_STREAMS */
static uint64_t         mc_gate_timeout_ns;

#define MC_HIP(call)                                                              \
    do {                                                                          \
        hipError_t e_ = (call);                                                   \
        if (e_ != hipSuccess && e_ != hipErrorDeinitialized) {                    \
            fprintf(stderr, "xccl mc_rocm: %s failed with %d (%s)\n", #call,      \
                    (int)e_, hipGetErrorString(e_));                              \
            return XCCL_ERR_NO_MESSAGE;                                           \
        }                                                                         \
    } while (0)

static int mc_rocm_backing_alloc(void **ptr, size_t len)
{
    hipError_t e = hipMalloc(ptr, len);

    if (e != hipSuccess) {
        (void)hipGetLastError(); /* leave no sticky error behind */
        return (int)e;
    }
    return 0;
}

static int mc_rocm_backing_free(void *ptr)
{
    hipError_t e = hipFree(ptr);

    if (e != hipSuccess && e != hipErrorDeinitialized) {
        (void)hipGetLastError();
        return (int)e;
    }
    return 0;
}

/* Environment knobs, read once: by open() when a loader calls it, else by the
 * first entry that needs them. */
static pthread_once_t mc_config_once = PTHREAD_ONCE_INIT;

static void mc_rocm_read_config(void)
{
    const char *s;
    size_t      pool_limit = MC_DEFAULT_POOL_MAX_BYTES;

    mc_graph_max_bytes = MC_DEFAULT_GRAPH_MAX_BYTES;
    s = getenv("XCCL_MC_ROCM_GRAPH_MAX_BYTES");
    if (s != NULL) {
        mc_graph_max_bytes = (size_t)strtoull(s, NULL, 0);
    }
    mc_gate_timeout_ns = (uint64_t)MC_DEFAULT_GATE_TIMEOUT_MS * 1000000ull;
    s = getenv("XCCL_MC_ROCM_GATE_TIMEOUT_MS");
    if (s != NULL) {
        mc_gate_timeout_ns = strtoull(s, NULL, 0) * 1000000ull;
    }
    s = getenv("XCCL_MC_ROCM_THREAD_STREAMS");
    if (s != NULL && atoi(s) >= 1 && atoi(s) <= MC_NUM_STREAMS) {
        mc_num_streams = atoi(s);
    }
    s = getenv("XCCL_MC_ROCM_POOL_MAX_BYTES");
    if (s != NULL) {
        pool_limit = (size_t)strtoull(s, NULL, 0);
    }
    mc_pool_configure(mc_rocm_backing_alloc, mc_rocm_backing_free, pool_limit);
}

static xccl_status_t mc_rocm_open(void)
{
    /* No device call here: the process may not have chosen its GPU yet. */
    (void)pthread_once(&mc_config_once, mc_rocm_read_config);
    return XCCL_OK;
}

/* Frees whatever of a device's resources exists; caller holds mc_init_lock
 * and has made that device current. */
static void mc_rocm_device_destroy(mc_rocm_device_t *d)
{
    int i;

    for (i = 0; i < XCCL_ROCM_MC_NUM_EVENTS; i++) {
        if (d->events[i].hip_event != NULL) {
            (void)hipEventDestroy(d->events[i].hip_event);
        }
    }
    for (i = 0; i < XCCL_ROCM_MC_NUM_STREAM_REQUESTS; i++) {
        if (d->requests[i].hip_event != NULL) {
            (void)hipEventDestroy(d->requests[i].hip_event);
        }
    }
    if (d->gate_words != NULL) {
        (void)hipHostFree(d->gate_words);
    }
    if (d->flag_words != NULL) {
        (void)hipHostFree(d->flag_words);
    }
    if (d->arrival_counts != NULL) {
        (void)hipFree(d->arrival_counts);
    }
    if (d->kernargs != NULL && d->kernargs_pinned) {
        (void)hipHostFree(d->kernargs);
    }
    for (i = 0; i < MC_NUM_STREAMS; i++) {
        if (d->stream[i] != NULL) {
            (void)hipStreamDestroy(d->stream[i]);
        }
    }
    memset(d, 0, sizeof(*d));
}

/* Stream, events and gate words of one device. */
static xccl_status_t mc_rocm_device_create_parts(mc_rocm_device_t *d)
{
    xccl_status_t st;
    int           i;

    MC_HIP(hipStreamCreateWithFlags(&d->stream[0], hipStreamNonBlocking));
    MC_HIP(hipHostMalloc((void **)&d->gate_words,
                         XCCL_ROCM_MC_NUM_STREAM_REQUESTS * sizeof(int),
                         hipHostMallocMapped));
    for (i = 0; i < XCCL_ROCM_MC_NUM_STREAM_REQUESTS; i++) {
        mc_rocm_stream_request_t *r = &d->requests[i];
        r->flag  = &d->gate_words[i];
        *r->flag = 1; /* open */
        MC_HIP(hipHostGetDevicePointer((void **)&r->dev_flag, r->flag, 0));
        MC_HIP(hipEventCreateWithFlags(&r->hip_event, hipEventDisableTiming));
        atomic_store(&r->is_free, MC_SLOT_FREE);
    }
    MC_HIP(hipHostMalloc((void **)&d->flag_words,
                         XCCL_ROCM_MC_NUM_EVENTS * MC_FLAG_STRIDE * sizeof(uint32_t),
                         hipHostMallocMapped));
    memset(d->flag_words, 0, XCCL_ROCM_MC_NUM_EVENTS * MC_FLAG_STRIDE * sizeof(uint32_t));
    MC_HIP(hipMalloc((void **)&d->arrival_counts,
                     XCCL_ROCM_MC_NUM_EVENTS * XCCL_ROCM_DONE_COUNT_BYTES));
    MC_HIP(hipMemsetAsync(d->arrival_counts, 0,
                          XCCL_ROCM_MC_NUM_EVENTS * XCCL_ROCM_DONE_COUNT_BYTES, d->stream[0]));
    MC_HIP(hipStreamSynchronize(d->stream[0]));
    /* compute-unit count, static counter array, the first of the component's own dispatch queues -- behind the
     * stream: a device serves its most recently created queue fastest (0.6 us per dispatch between the newest and
     * an older one, measured) */
    st = xccl_rocm_prepare_device();
    if (st != XCCL_OK) {
        return st;
    }
    d->kernargs = (char *)xccl_rocm_direct_kernarg_arena(XCCL_ROCM_MC_NUM_EVENTS * XCCL_ROCM_KERNARG_BYTES);
    if (d->kernargs == NULL) {
        MC_HIP(hipHostMalloc((void **)&d->kernargs, XCCL_ROCM_MC_NUM_EVENTS * XCCL_ROCM_KERNARG_BYTES, hipHostMallocDefault));
        memset(d->kernargs, 0, XCCL_ROCM_MC_NUM_EVENTS * XCCL_ROCM_KERNARG_BYTES);
        d->kernargs_pinned = 1;
    }
    for (i = 0; i < XCCL_ROCM_MC_NUM_EVENTS; i++) {
        mc_rocm_event_t *ev = &d->events[i];
        ev->kernarg = d->kernargs + (size_t)i * XCCL_ROCM_KERNARG_BYTES;
        ev->signal  = 0;
        MC_HIP(hipEventCreateWithFlags(&ev->hip_event, hipEventDisableTiming));
        ev->flag = &d->flag_words[i * MC_FLAG_STRIDE];
        MC_HIP(hipHostGetDevicePointer((void **)&ev->dev_flag, (void *)ev->flag, 0));
        ev->dev_count = d->arrival_counts + (size_t)i * (XCCL_ROCM_DONE_COUNT_BYTES / sizeof(uint32_t));
        ev->expect    = 0;
        ev->flagged   = 0;
        atomic_store(&ev->is_free, MC_SLOT_FREE);
    }
    return XCCL_OK;
}

/* All or nothing: a device whose set-up failed half-way keeps no resources and
 * is tried again on the next call.  Caller holds mc_init_lock. */
static xccl_status_t mc_rocm_device_create(mc_rocm_device_t *d)
{
    xccl_status_t st = mc_rocm_device_create_parts(d);

    if (st != XCCL_OK) {
        mc_rocm_device_destroy(d);
    }
    return st;
}

/* The current device's resources, created on first use. */
static xccl_status_t mc_rocm_device(mc_rocm_device_t **out)
{
    int               dev = 0;
    mc_rocm_device_t *d;
    xccl_status_t     st = XCCL_OK;

    (void)pthread_once(&mc_config_once, mc_rocm_read_config);
    MC_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= MC_MAX_DEVICES) {
        return XCCL_ERR_NO_RESOURCE;
    }
    d = &mc_devices[dev];
    if (atomic_load_explicit(&d->ready, memory_order_acquire) == 0) {
        pthread_mutex_lock(&mc_init_lock);
        if (atomic_load_explicit(&d->ready, memory_order_relaxed) == 0) {
            st = mc_rocm_device_create(d);
            if (st == XCCL_OK) {
                atomic_store_explicit(&d->ready, 1, memory_order_release);
            }
        }
        pthread_mutex_unlock(&mc_init_lock);
    }
    *out = d;
    return st;
}

/* The current device's resources for work that goes into the caller's stream.
 * Creating them allocates and synchronises, which would invalidate a capture
 * in progress: a first call on a device must not come from inside one. */
static xccl_status_t mc_rocm_device_for_stream(mc_rocm_device_t **out, hipStream_t hs)
{
    int                    dev = 0;
    hipStreamCaptureStatus cs  = hipStreamCaptureStatusNone;

    if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < MC_MAX_DEVICES &&
        atomic_load_explicit(&mc_devices[dev].ready, memory_order_acquire) == 0 &&
        hipStreamIsCapturing(hs, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone) {
        fprintf(stderr, "xccl mc_rocm: first use of device %d inside a stream capture; call any entry of the "
                        "component once outside the capture first\n", dev);
        return XCCL_ERR_NO_RESOURCE;
    }
    return mc_rocm_device(out);
}

/* The reduction stream of the calling thread on this device: every thread
 * sticks to one of mc_num_streams streams, handed out round-robin at its first
 * call; streams beyond the first are created when a thread first needs one. */
static unsigned mc_rocm_thread_index(void)
{
    static atomic_uint       next_index;
    static _Thread_local int index = -1;

    if (index < 0) {
        index = (int)(atomic_fetch_add(&next_index, 1) & 0x7fffffffu);
    }
    return (unsigned)index;
}

static int mc_rocm_thread_slot(void)
{
    return (int)(mc_rocm_thread_index() % (unsigned)mc_num_streams);
}

static xccl_status_t mc_rocm_thread_stream(mc_rocm_device_t *d, hipStream_t *out)
{
    const int     slot = mc_rocm_thread_slot();
    xccl_status_t st   = XCCL_OK;

    if (__atomic_load_n(&d->stream[slot], __ATOMIC_ACQUIRE) == NULL) {
        pthread_mutex_lock(&mc_init_lock);
        if (d->stream[slot] == NULL) {
            hipStream_t hs = NULL;
            if (hipStreamCreateWithFlags(&hs, hipStreamNonBlocking) != hipSuccess) {
                (void)hipGetLastError();
                st = XCCL_ERR_NO_MESSAGE;
            } else {
                __atomic_store_n(&d->stream[slot], hs, __ATOMIC_RELEASE);
            }
        }
        pthread_mutex_unlock(&mc_init_lock);
    }
    *out = d->stream[slot];
    return st;
}

/* cuda_mem_component.c:34-44, with freed blocks cached (mc_pool.h). */
static xccl_status_t mc_rocm_mem_alloc(void **ptr, size_t len)
{
    int dev = 0, rc;

    (void)pthread_once(&mc_config_once, mc_rocm_read_config);
    MC_HIP(hipGetDevice(&dev));
    rc = mc_pool_alloc(dev, ptr, len);
    if (rc != 0) {
        fprintf(stderr, "xccl mc_rocm: device allocation of %zu bytes failed with %d (%s)\n", len, rc,
                hipGetErrorString((hipError_t)rc));
        return XCCL_ERR_NO_MESSAGE;
    }
    return XCCL_OK;
}

/* The block goes back to the cache, not to the runtime, so the implicit device
 * synchronisation of the reference's cudaFree (cuda_mem_component.c:40-44) is
 * gone: free a block only after all work that touches it has completed, or the
 * next mem_alloc may hand it out while that work still runs. */
static xccl_status_t mc_rocm_mem_free(void *ptr)
{
    int rc;

    (void)pthread_once(&mc_config_once, mc_rocm_read_config);
    rc = mc_pool_free(ptr);
    if (rc != 0) {
        fprintf(stderr, "xccl mc_rocm: mem_free(%p) failed with %d%s\n", ptr, rc,
                rc < 0 ? " (block freed twice)" : "");
        return XCCL_ERR_NO_MESSAGE;
    }
    return XCCL_OK;
}

void xccl_rocm_mem_pool_set_limit(size_t limit_bytes)
{
    (void)pthread_once(&mc_config_once, mc_rocm_read_config);
    mc_pool_set_limit(limit_bytes);
}

void xccl_rocm_mem_pool_get_stats(xccl_rocm_mem_pool_stats_t *out)
{
    mc_pool_stats_t st;

    mc_pool_get_stats(&st);
    out->hits          = st.hits;
    out->misses        = st.misses;
    out->backing_frees = st.backing_frees;
    out->cached_bytes  = st.cached_bytes;
    out->live_blocks   = st.live_blocks;
    out->free_blocks   = st.free_blocks;
}

/* cuda_mem_component.c:182-204: device memory -> this component's type,
 * every other pointer the runtime knows (pinned host, managed) -> HOST, a
 * pointer it does not know -> XCCL_ERR_UNSUPPORTED with the runtime's sticky
 * error cleared. */
static xccl_status_t mc_rocm_mem_type(void *ptr, ucs_memory_type_t *mem_type)
{
    hipPointerAttribute_t attr;
    hipError_t            err;

    err = hipPointerGetAttributes(&attr, ptr);
    if (err != hipSuccess) {
        (void)hipGetLastError();
        return XCCL_ERR_UNSUPPORTED;
    }
    if (attr.type == hipMemoryTypeDevice) {
        *mem_type = UCS_MEMORY_TYPE_ROCM;
    } else {
        *mem_type = UCS_MEMORY_TYPE_HOST;
    }
    return XCCL_OK;
}

/* The last launch the calling thread put on the component's own dispatch queue
 * without waiting for it.  Launches of that queue and of the thread's HIP
 * stream are not ordered against each other by the device, so the thread's
 * next launch on the stream waits for this one on the host first (rare: a
 * small stream-ordered reduction followed by a large one). */
static _Thread_local struct {
    volatile uint32_t *flag;
    int                words; /* -1: complete when `signal` reads 0 */
    uint32_t           expect;
    uint64_t           signal;
    unsigned           generation;
} mc_last_direct;

/* bumped by close(): completion words recorded before it are gone */
static atomic_uint mc_generation;

static void mc_rocm_wait_last_direct(void)
{
    unsigned polls = 0;
    int      i;

    if (mc_last_direct.flag == NULL) {
        return;
    }
    if (mc_last_direct.generation != atomic_load(&mc_generation)) {
        mc_last_direct.flag = NULL;
        return;
    }
    while (mc_last_direct.words < 0 && !xccl_rocm_direct_signal_done(mc_last_direct.signal)) {
        /* (a later launch of the same event re-arms the signal only after this one was seen complete) */
        if ((++polls & 0xffffu) == 0 && xccl_rocm_direct_queue_failed()) {
            break;
        }
        MC_CPU_RELAX();
    }
    for (i = 0; i < mc_last_direct.words; i++) {
        /* sequence numbers of a word only grow: at or past ours means ours is done */
        while ((int32_t)(__atomic_load_n(&mc_last_direct.flag[i], __ATOMIC_ACQUIRE) - mc_last_direct.expect) < 0) {
            if ((++polls & 0xffffu) == 0 && xccl_rocm_direct_queue_failed()) {
                break;
            }
            MC_CPU_RELAX();
        }
    }
    mc_last_direct.flag = NULL;
}

static int mc_rocm_stream_idle(mc_rocm_device_t *d, int slot)
{
    return atomic_load_explicit(&d->stream_issued[slot], memory_order_acquire) ==
           atomic_load_explicit(&d->stream_synced[slot], memory_order_acquire);
}

/* A launch on a reduction stream has been seen complete: so have all before it. */
static void mc_rocm_note_complete(mc_rocm_event_t *ev)
{
    unsigned seen;

    if (ev->direct || ev->slot < 0 || ev->dev == NULL) {
        return;
    }
    seen = atomic_load_explicit(&ev->dev->stream_synced[ev->slot], memory_order_relaxed);
    while ((int)(ev->stream_seq - seen) > 0 &&
           !atomic_compare_exchange_weak(&ev->dev->stream_synced[ev->slot], &seen, ev->stream_seq)) {
    }
}

/* Whether the flagged launch an event stands for has completed. */
static int mc_rocm_flag_done(const mc_rocm_event_t *ev)
{
    int i;

    if (ev->flagged < 0) {
        return xccl_rocm_direct_signal_done(ev->signal);
    }
    for (i = 0; i < ev->flagged; i++) {
        if (__atomic_load_n(&ev->flag[i], __ATOMIC_ACQUIRE) != ev->expect) {
            return 0;
        }
    }
    return 1;
}

static mc_rocm_event_t *mc_rocm_claim_event(mc_rocm_device_t *d)
{
    /* threads start their search in different quarters of the pool, so that
     * they do not all fight for the first slots */
    const unsigned first = (mc_rocm_thread_index() % 4u) * (XCCL_ROCM_MC_NUM_EVENTS / 4u);
    int            i, expect;

    for (i = 0; i < XCCL_ROCM_MC_NUM_EVENTS; i++) {
        mc_rocm_event_t *ev = &d->events[(first + (unsigned)i) % XCCL_ROCM_MC_NUM_EVENTS];
        expect = MC_SLOT_FREE;
        if (!atomic_compare_exchange_strong(&ev->is_free, &expect, MC_SLOT_BUSY)) {
            continue;
        }
        if (ev->flagged && !mc_rocm_flag_done(ev)) {
            /* freed by its owner before the launch it stands for finished: its
             * completion word and arrival counter are still in use */
            atomic_store(&ev->is_free, MC_SLOT_FREE);
            continue;
        }
        return ev;
    }
    return NULL;
}

static xccl_status_t mc_rocm_user_stream(xccl_stream_t *stream, hipStream_t *out)
{
    if (stream == NULL || stream->stream == NULL) {
        return XCCL_ERR_INVALID_PARAM;
    }
    *out = *(hipStream_t *)stream->stream;
    return XCCL_OK;
}

/* Completion of a flagged launch, observed from the host.  `block`: spin until
 * done.  Every 64 Ki polls the stream is asked whether it failed or drained
 * without the word being written (a launch on the component's own queue: whether
 * that queue reported an error), so a broken launch cannot spin forever. */
static xccl_status_t mc_rocm_flag_poll(mc_rocm_event_t *ev, int block)
{
    hipError_t e;

    for (;;) {
        if (mc_rocm_flag_done(ev)) {
            mc_rocm_note_complete(ev);
            return XCCL_OK;
        }
        if ((++ev->polls & 0xffffu) == 0 && ev->direct) {
            if (xccl_rocm_direct_queue_failed()) {
                return XCCL_ERR_NO_MESSAGE;
            }
        } else if ((ev->polls & 0xffffu) == 0) {
            e = hipStreamQuery(ev->stream);
            if (e == hipSuccess) {
                return mc_rocm_flag_done(ev) ? XCCL_OK : XCCL_ERR_NO_MESSAGE;
            }
            if (e != hipErrorNotReady) {
                return XCCL_ERR_NO_MESSAGE;
            }
        }
        if (!block) {
            return XCCL_INPROGRESS;
        }
        MC_CPU_RELAX();
    }
}

/* Shared tail of the four reduction entries.  `want_sync`: block until the
 * result is visible (the vtable's reduce / reduce_multi contract, reference
 * xccl_cuda_reduce_multi.cu:140). */
static xccl_status_t mc_rocm_do_reduce_multi(void *sbuf1, void *sbuf2,
                                             void *rbuf, size_t count,
                                             size_t size, size_t stride,
                                             xccl_dt_t dtype, xccl_op_t op,
                                             xccl_stream_t *stream,
                                             xccl_mc_event_t **event,
                                             int want_sync)
{
    mc_rocm_device_t *d;
    mc_rocm_event_t  *ev = NULL;
    hipStream_t       hs;
    xccl_status_t     st;
    int               flagged = 0, slot;
    unsigned          stream_seq = 0;

    st = xccl_rocm_reduce_supported(dtype, op);
    if (st != XCCL_OK) {
        return st;
    }
    if (stream != NULL) {
        st = mc_rocm_user_stream(stream, &hs);
        if (st != XCCL_OK) {
            return st;
        }
        st = mc_rocm_device_for_stream(&d, hs);
    } else {
        st = mc_rocm_device(&d);
        if (st == XCCL_OK) {
            /* created now even if this call ends up on the component's own dispatch queue: that queue is
             * created after it, and a device serves its most recently created queue fastest */
            st = mc_rocm_thread_stream(d, &hs);
        }
    }
    if (st != XCCL_OK) {
        return st;
    }
    if (event != NULL || want_sync) {
        /* a pooled event brings the completion word; a blocking call can do
         * without one (then it waits for the stream) */
        ev = mc_rocm_claim_event(d);
        if (ev == NULL && event != NULL) {
            return XCCL_ERR_NO_RESOURCE;
        }
    }

    slot = stream == NULL ? mc_rocm_thread_slot() : -1;
    if (slot >= 0 && ev != NULL && mc_graph_max_bytes == 0 && mc_rocm_stream_idle(d, slot)) {
        /* The launch will tell its own completion, and this slot's stream holds
         * nothing to stay behind: it needs no stream at all.  The component's
         * own queue runs this slot's launches in order. */
        st = xccl_rocm_reduce_multi_direct(sbuf1, sbuf2, rbuf, count, size,
                                           stride, dtype, op, slot,
                                           ev->dev_count, ev->dev_flag,
                                           MC_FLAG_STRIDE, ev->expect + 1,
                                           &ev->signal, ev->kernarg,
                                           want_sync && mc_last_direct.flag == NULL,
                                           &flagged);
        if (st != XCCL_OK) {
            atomic_store(&ev->is_free, MC_SLOT_FREE);
            return st;
        }
        if (flagged) {
            ev->stream  = hs;
            ev->flagged = flagged;
            ev->direct  = 1;
            ev->slot    = -1;
            ev->polls   = 0;
            if (flagged > 0) {
                ev->expect++;
            }
            if (want_sync) {
                st = mc_rocm_flag_poll(ev, 1);
            } else {
                mc_last_direct.flag       = ev->flag;
                mc_last_direct.words      = flagged;
                mc_last_direct.expect     = ev->expect;
                mc_last_direct.signal     = ev->signal;
                mc_last_direct.generation = atomic_load(&mc_generation);
            }
            if (event != NULL && st == XCCL_OK) {
                ev->super.mem_type = UCS_MEMORY_TYPE_ROCM;
                *event             = &ev->super;
            } else {
                atomic_store(&ev->is_free, MC_SLOT_FREE);
            }
            return st;
        }
    }
    if (slot >= 0) {
        mc_rocm_wait_last_direct();
    }
    if (want_sync && size * xccl_dt_size(dtype) <= mc_graph_max_bytes) {
        st = xccl_rocm_reduce_multi_graph(sbuf1, sbuf2, rbuf, count, size,
                                          stride, dtype, op, hs);
    } else if (ev != NULL) {
        st = xccl_rocm_reduce_multi_slots(sbuf1, sbuf2, rbuf, count, size,
                                          stride, dtype, op, hs,
                                          ev->dev_count, ev->dev_flag,
                                          MC_FLAG_STRIDE, ev->expect + 1,
                                          &flagged);
    } else {
        st = xccl_rocm_reduce_multi_impl(sbuf1, sbuf2, rbuf, count, size,
                                         stride, dtype, op, hs);
    }
    if (st != XCCL_OK) {
        if (ev != NULL) {
            atomic_store(&ev->is_free, MC_SLOT_FREE);
        }
        return st;
    }
    if (slot >= 0) {
        stream_seq = atomic_fetch_add_explicit(&d->stream_issued[slot], 1, memory_order_acq_rel) + 1;
    }
    if (ev != NULL) {
        ev->stream     = hs;
        ev->flagged    = flagged;
        ev->direct     = 0;
        ev->slot       = slot;
        ev->stream_seq = stream_seq;
        ev->dev        = d;
        ev->polls      = 0;
        if (flagged) {
            ev->expect++;
        } else if (event != NULL && hipEventRecord(ev->hip_event, hs) != hipSuccess) {
            atomic_store(&ev->is_free, MC_SLOT_FREE);
            return XCCL_ERR_NO_MESSAGE;
        }
    }
    if (want_sync) {
        if (flagged) {
            st = mc_rocm_flag_poll(ev, 1);
        } else if (hipStreamSynchronize(hs) != hipSuccess) {
            st = XCCL_ERR_NO_MESSAGE;
        } else if (ev != NULL) {
            mc_rocm_note_complete(ev);
        } else if (slot >= 0) {
            mc_rocm_event_t none = {.direct = 0, .slot = slot, .stream_seq = stream_seq, .dev = d};
            mc_rocm_note_complete(&none);
        }
    }
    if (ev != NULL) {
        if (event != NULL && st == XCCL_OK) {
            ev->super.mem_type = UCS_MEMORY_TYPE_ROCM;
            *event             = &ev->super;
        } else {
            atomic_store(&ev->is_free, MC_SLOT_FREE);
        }
    }
    return st;
}

static xccl_status_t mc_rocm_reduce(void *sbuf1, void *sbuf2, void *target,
                                    size_t count, xccl_dt_t dtype, xccl_op_t op)
{
    return mc_rocm_do_reduce_multi(sbuf1, sbuf2, target, 1, count, 0, dtype, op,
                                   NULL, NULL, 1);
}

static xccl_status_t mc_rocm_reduce_multi(void *sbuf1, void *sbuf2, void *rbuf,
                                          size_t count, size_t size,
                                          size_t stride, xccl_dt_t dtype,
                                          xccl_op_t op)
{
    return mc_rocm_do_reduce_multi(sbuf1, sbuf2, rbuf, count, size, stride,
                                   dtype, op, NULL, NULL, 1);
}

static xccl_status_t mc_rocm_reduce_nb(void *sbuf1, void *sbuf2, void *target,
                                       size_t count, xccl_dt_t dtype,
                                       xccl_op_t op, xccl_stream_t *stream,
                                       xccl_mc_event_t **event)
{
    return mc_rocm_do_reduce_multi(sbuf1, sbuf2, target, 1, count, 0, dtype, op,
                                   stream, event, 0);
}

static xccl_status_t mc_rocm_reduce_multi_nb(void *sbuf1, void *sbuf2,
                                             void *rbuf, size_t count,
                                             size_t size, size_t stride,
                                             xccl_dt_t dtype, xccl_op_t op,
                                             xccl_stream_t *stream,
                                             xccl_mc_event_t **event)
{
    return mc_rocm_do_reduce_multi(sbuf1, sbuf2, rbuf, count, size, stride,
                                   dtype, op, stream, event, 0);
}

/* Note the argument order: source first (mem_component.h:38). */
static xccl_status_t mc_rocm_memcpy_async(void *sbuf, void *dbuf, size_t size,
                                          xccl_stream_t *stream)
{
    hipStream_t   hs;
    xccl_status_t st = mc_rocm_user_stream(stream, &hs);

    if (st != XCCL_OK) {
        return st;
    }
    MC_HIP(hipMemcpyAsync(dbuf, sbuf, size, hipMemcpyDefault, hs));
    return XCCL_OK;
}

static xccl_status_t mc_rocm_event_record(xccl_stream_t *stream,
                                          xccl_mc_event_t **event)
{
    mc_rocm_device_t *d;
    mc_rocm_event_t  *ev;
    hipStream_t       hs;
    hipError_t        e;
    xccl_status_t     st;

    st = mc_rocm_user_stream(stream, &hs);
    if (st != XCCL_OK) {
        return st;
    }
    st = mc_rocm_device_for_stream(&d, hs);
    if (st != XCCL_OK) {
        return st;
    }
    ev = mc_rocm_claim_event(d);
    if (ev == NULL) {
        return XCCL_ERR_NO_RESOURCE;
    }
    ev->flagged = 0;
    ev->direct  = 0;
    ev->slot    = -1;
    ev->stream  = hs;
    e = hipEventRecord(ev->hip_event, hs);
    if (e != hipSuccess) {
        atomic_store(&ev->is_free, MC_SLOT_FREE);
        return XCCL_ERR_NO_MESSAGE;
    }
    ev->super.mem_type = UCS_MEMORY_TYPE_ROCM;
    *event             = &ev->super;
    return XCCL_OK;
}

static mc_rocm_event_t *mc_rocm_event_of(xccl_mc_event_t *event)
{
    return (mc_rocm_event_t *)((char *)event - offsetof(mc_rocm_event_t, super));
}

static xccl_status_t mc_rocm_event_query(xccl_mc_event_t *event)
{
    hipError_t e;

    if (event == NULL) {
        return XCCL_ERR_INVALID_PARAM;
    }
    if (mc_rocm_event_of(event)->flagged) {
        return mc_rocm_flag_poll(mc_rocm_event_of(event), 0);
    }
    e = hipEventQuery(mc_rocm_event_of(event)->hip_event);
    if (e == hipSuccess) {
        mc_rocm_note_complete(mc_rocm_event_of(event));
        return XCCL_OK;
    }
    if (e == hipErrorNotReady) {
        return XCCL_INPROGRESS;
    }
    return XCCL_ERR_NO_MESSAGE;
}

static xccl_status_t mc_rocm_event_wait(xccl_mc_event_t *event)
{
    if (event == NULL) {
        return XCCL_ERR_INVALID_PARAM;
    }
    if (mc_rocm_event_of(event)->flagged) {
        return mc_rocm_flag_poll(mc_rocm_event_of(event), 1);
    }
    MC_HIP(hipEventSynchronize(mc_rocm_event_of(event)->hip_event));
    mc_rocm_note_complete(mc_rocm_event_of(event));
    return XCCL_OK;
}

static xccl_status_t mc_rocm_event_free(xccl_mc_event_t *event)
{
    if (event == NULL) {
        return XCCL_ERR_INVALID_PARAM;
    }
    atomic_store(&mc_rocm_event_of(event)->is_free, MC_SLOT_FREE);
    return XCCL_OK;
}

/* cuda_mem_component.c:139-162: block the USER's stream until the host calls
 * finish_stream_activity.  A gate kernel that polls a host-mapped word goes
 * straight into the user's stream.  The reference puts its spin kernel on the
 * stream its reductions use and lets the user's stream wait for an event behind
 * it: a reduction issued while the gate is shut then waits for the very
 * collective that is waiting for the reduction, gates of different user
 * streams wait for each other, and two hardware queues are held up instead of
 * one.  (Streams that share the user's hardware queue -- a process has 4 by
 * default -- are still held up while a gate is shut; the gate's wait is
 * bounded.) */
static xccl_status_t
mc_rocm_start_stream_activity(xccl_stream_t *stream,
                              xccl_mem_component_stream_request_t **req)
{
    mc_rocm_device_t         *d;
    mc_rocm_stream_request_t *r = NULL;
    hipStream_t               user;
    xccl_status_t             st;
    int                       i, expect;

    st = mc_rocm_user_stream(stream, &user);
    if (st != XCCL_OK) {
        return st;
    }
    st = mc_rocm_device_for_stream(&d, user);
    if (st != XCCL_OK) {
        return st;
    }
    for (i = 0; i < XCCL_ROCM_MC_NUM_STREAM_REQUESTS && r == NULL; i++) {
        expect = MC_SLOT_FREE;
        if (atomic_compare_exchange_strong(&d->requests[i].is_free, &expect,
                                           MC_SLOT_BUSY)) {
            r = &d->requests[i];
        } else if (expect == MC_SLOT_DRAINING &&
                   hipEventQuery(d->requests[i].hip_event) == hipSuccess &&
                   atomic_compare_exchange_strong(&d->requests[i].is_free,
                                                  &expect, MC_SLOT_BUSY)) {
            r = &d->requests[i]; /* its previous gate kernel has retired */
        }
    }
    if (r == NULL) {
        return XCCL_ERR_NO_RESOURCE;
    }
    __atomic_store_n(r->flag, 0, __ATOMIC_RELEASE);
    st = xccl_rocm_stream_gate(r->dev_flag, mc_gate_timeout_ns, user);
    if (st != XCCL_OK) {
        atomic_store(&r->is_free, MC_SLOT_FREE);
        return st;
    }
    if (hipEventRecord(r->hip_event, user) != hipSuccess) { /* tells when the gate kernel has retired */
        /* open the gate again: nothing may stay blocked behind a failure */
        __atomic_store_n(r->flag, 1, __ATOMIC_RELEASE);
        atomic_store(&r->is_free, MC_SLOT_FREE);
        return XCCL_ERR_NO_MESSAGE;
    }
    r->super.mem_type = UCS_MEMORY_TYPE_ROCM;
    *req              = &r->super;
    return XCCL_OK;
}

static xccl_status_t
mc_rocm_finish_stream_activity(xccl_mem_component_stream_request_t *req)
{
    mc_rocm_stream_request_t *r;
    int                       old;

    if (req == NULL) {
        return XCCL_ERR_INVALID_PARAM;
    }
    r = (mc_rocm_stream_request_t *)((char *)req -
                                     offsetof(mc_rocm_stream_request_t, super));
    old = __atomic_exchange_n(r->flag, 1, __ATOMIC_ACQ_REL);
    /* Not reusable until its gate kernel has seen the word and left the
     * queue; start_stream_activity checks that when it claims the slot. */
    atomic_store(&r->is_free, MC_SLOT_DRAINING);
    if (old == 2) {
        /* the gate kernel ran into its time limit and let the user's stream go
         * on before the collective had finished: stream order was not kept */
        fprintf(stderr, "xccl mc_rocm: stream gate gave up after %llu ms (XCCL_MC_ROCM_GATE_TIMEOUT_MS) before "
                        "finish_stream_activity; work queued behind it ran early\n",
                (unsigned long long)(mc_gate_timeout_ns / 1000000ull));
        return XCCL_ERR_NO_PROGRESS;
    }
    return XCCL_OK;
}

static xccl_status_t mc_rocm_get_stream(void **hip_stream)
{
    mc_rocm_device_t *d;
    xccl_status_t     st = mc_rocm_device(&d);

    if (st != XCCL_OK) {
        return st;
    }
    st = mc_rocm_thread_stream(d, (hipStream_t *)hip_stream);
    if (st != XCCL_OK) {
        return st;
    }
    return XCCL_OK;
}

/* Releases the resources of every device that was used.  (The reference
 * component owns one device's worth, cuda_mem_component.c:251-265; this one
 * keeps a set per device ordinal, so close visits each.) */
static void mc_rocm_close(void)
{
    mc_rocm_device_t *d;
    int               cur = 0, dev, i;

    if (hipGetDevice(&cur) != hipSuccess) {
        (void)hipGetLastError();
        return;
    }
    mc_pool_trim(-1);
    atomic_fetch_add(&mc_generation, 1);
    pthread_mutex_lock(&mc_init_lock);
    for (dev = 0; dev < MC_MAX_DEVICES; dev++) {
        d = &mc_devices[dev];
        if (atomic_load(&d->ready) != 1) {
            continue;
        }
        if (hipSetDevice(dev) != hipSuccess) {
            (void)hipGetLastError();
            continue;
        }
        for (i = 0; i < XCCL_ROCM_MC_NUM_STREAM_REQUESTS; i++) {
            __atomic_store_n(d->requests[i].flag, 1, __ATOMIC_RELEASE); /* open any gate left shut */
        }
        for (i = 0; i < XCCL_ROCM_MC_NUM_STREAM_REQUESTS; i++) {
            if (atomic_load(&d->requests[i].is_free) != MC_SLOT_FREE) {
                (void)hipEventSynchronize(d->requests[i].hip_event); /* its gate kernel has left the queue */
            }
        }
        for (i = 0; i < MC_NUM_STREAMS; i++) {
            if (d->stream[i] != NULL) {
                (void)hipStreamSynchronize(d->stream[i]);
            }
        }
        xccl_rocm_graph_cache_destroy();
        xccl_rocm_direct_queue_destroy();
        mc_rocm_device_destroy(d); /* also clears `ready` */
    }
    (void)hipSetDevice(cur);
    pthread_mutex_unlock(&mc_init_lock);
}

xccl_rocm_mem_component_t xccl_rocm_mem_component = {
    .super = {
        .open                   = mc_rocm_open,
        .mem_alloc              = mc_rocm_mem_alloc,
        .mem_free               = mc_rocm_mem_free,
        .mem_type               = mc_rocm_mem_type,
        .reduce                 = mc_rocm_reduce,
        .reduce_multi           = mc_rocm_reduce_multi,
        .memcpy_async           = mc_rocm_memcpy_async,
        .event_record           = mc_rocm_event_record,
        .event_query            = mc_rocm_event_query,
        .event_free             = mc_rocm_event_free,
        .start_stream_activity  = mc_rocm_start_stream_activity,
        .finish_stream_activity = mc_rocm_finish_stream_activity,
        .close                  = mc_rocm_close,
    },
    .ext_version     = XCCL_ROCM_MC_EXT_VERSION,
    .reduce_nb       = mc_rocm_reduce_nb,
    .reduce_multi_nb = mc_rocm_reduce_multi_nb,
    .event_wait      = mc_rocm_event_wait,
    .get_stream      = mc_rocm_get_stream,
};

/* How a loader learns that this component has the extension without reading
 * past a foreign component's vtable: a second data symbol pointing at it. */
xccl_rocm_mem_component_t *const xccl_rocm_mem_component_ext = &xccl_rocm_mem_component;

/* The reference loader asks every component file for this one name
 * (src/utils/mem_component.c:30). */
extern xccl_rocm_mem_component_t xccl_cuda_mem_component
    __attribute__((alias("xccl_rocm_mem_component")));
