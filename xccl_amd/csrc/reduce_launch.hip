// reduce_launch.hip -- host side of the kernel ABI declared in
// include/xccl_rocm_kernels.h: (dtype, op) -> kernel lookup, launch planning,
// plain launch, the cached single-node hipGraph launch, and the stream gate.
#include "reduce_kernel.hpp"
#include "xccl_rocm_kernels.h"

#include <hsa/hsa.h>
#include <hsa/hsa_ext_amd.h>

#include <atomic>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

namespace xccl_rocm {
namespace {

constexpr int kMaxDevices       = 64;
// Grid cap in workgroups per compute unit.  Large on purpose: one tile per
// workgroup measured fastest, so the cap only bounds the grid of huge calls.
constexpr int kDefaultBlocksPerCu = 8192;

// Resident one-wave workgroups per compute unit for large launches (0 = the
// defaults of lds_for_resident, > 0 = this many for every call,
// >= kNoResidentCap = no cap).
constexpr int    kNoResidentCap = 32;
constexpr size_t kLdsPerCu      = 160 * 1024;
constexpr size_t kLdsPerGroup   = 64 * 1024; // most a workgroup may ask for

// Launches of at most this many workgroups may count their own arrivals for a
// completion word: each workgroup pays an atomic on one of 64 shared counters
// (~12 ns per arrival on the same word, measured), which beats the queue's
// completion signal up to here and would serialise a grid of hundreds of
// thousands.
constexpr unsigned kMaxFlaggedGrid = 8192;
// Hard bound of what XCCL_MC_ROCM_MAX_COUNTED_GRID may ask for (measurement; the two-level count itself has no limit).
constexpr unsigned kMaxCountedGridKnob = 1u << 20;

std::atomic<int> g_blocks_per_cu{-1}; // -1: not read from the environment yet
std::atomic<int> g_resident{0};
std::atomic<int> g_tail_flag{1};
std::atomic<unsigned> g_shape_epoch{0}; // bumped when a launch-shape knob changes
// the same bound for launches on the component's own dispatch queue, where the alternative to counting is the
// stream path as a whole (blocking call, us, counting on the own queue / queued kernel on the stream: 3072
// workgroups 7.8 / 8.8-9.3, 4096: 8.2 / 8.9-9.4, 6144: 9.2 / 9.2-9.4, 8192: 10.0 / 9.6-9.8)
std::atomic<unsigned> g_direct_counted_grid{6144};
std::atomic<unsigned> g_max_counted_grid{2048}; // measured (blocking call, us, counting / queued kernel): 512 workgroups 8.0 / 9.2, 2048: 8.6-9.7 / 9.4-9.5, 8192: 10.4 / 10.0
// Launches of at most this many workgroups (and at least 4 sources; up to 3 the
// walk has every load in flight anyway) use the burst kernel: all loads of a
// tile at once.  Such a launch leaves the memory side idle and is bound by the
// chain of load latencies, which the walk makes as long as half the source count.
// Measured, blocking call, fp32 SUM, us (walk / burst): 8 sources x 1 KiB 6.73 / 6.51,
// x 32 KiB 8.00 / 7.78, x 2 MiB 9.57 / 9.29, x 4 MiB 11.35 / 11.27, x 16 MiB 28.9 / 30.6;
// 16 sources x 1 KiB 7.39 / 6.89, x 512 KiB 10.50 / 9.16, x 2 MiB 11.94 / 10.92,
// x 4 MiB 16.45 / 18.14; 4 sources: equal up to 2 MiB, the walk ahead beyond.
std::atomic<unsigned> g_burst_max_grid{2048};
// Launches of at most this many workgroups report completion on one word per
// workgroup when the caller has room for them (see xccl_rocm_reduce_multi_slots).
constexpr unsigned kDefaultSlotMaxGrid = 8; // measured: see xccl_rocm_reduce_multi_slots in the header
std::atomic<unsigned> g_slot_max_grid{kDefaultSlotMaxGrid};
std::atomic<int> g_cu_count[kMaxDevices];

void read_env_once()
{
    if (g_blocks_per_cu.load(std::memory_order_acquire) >= 0) {
        return;
    }
    const char *bpc = getenv("XCCL_MC_ROCM_BLOCKS_PER_CU");
    const char *res = getenv("XCCL_MC_ROCM_RESIDENT_PER_CU");
    const char *tf  = getenv("XCCL_MC_ROCM_TAIL_FLAG");
    g_tail_flag.store(tf ? atoi(tf) != 0 : 1, std::memory_order_release);
    const char *bmg = getenv("XCCL_MC_ROCM_BURST_MAX_GRID");
    if (bmg != nullptr && atoi(bmg) >= 0) {
        g_burst_max_grid.store((unsigned)atoi(bmg), std::memory_order_release);
    }
    const char *smg = getenv("XCCL_MC_ROCM_SLOT_MAX_GRID");
    if (smg != nullptr && atoi(smg) >= 0) {
        g_slot_max_grid.store((unsigned)atoi(smg), std::memory_order_release);
    }
    const char *mcg = getenv("XCCL_MC_ROCM_MAX_COUNTED_GRID");
    if (mcg != nullptr && atoi(mcg) >= 0 && (unsigned)atoi(mcg) <= kMaxCountedGridKnob) {
        g_max_counted_grid.store((unsigned)atoi(mcg), std::memory_order_release);
        g_direct_counted_grid.store((unsigned)atoi(mcg), std::memory_order_release);
    }
    int         v   = bpc ? atoi(bpc) : 0;
    g_resident.store(res && atoi(res) > 0 ? atoi(res) : 0, std::memory_order_release);
    g_blocks_per_cu.store(v > 0 ? v : kDefaultBlocksPerCu, std::memory_order_release);
}

// Compute units of the current device (cached per device ordinal).
xccl_status_t cu_count(int *cus)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        return XCCL_ERR_NO_MESSAGE;
    }
    if (dev < 0 || dev >= kMaxDevices) {
        return XCCL_ERR_NO_RESOURCE;
    }
    int n = g_cu_count[dev].load(std::memory_order_acquire);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            return XCCL_ERR_NO_MESSAGE;
        }
        g_cu_count[dev].store(n, std::memory_order_release);
    }
    *cus = n;
    return XCCL_OK;
}

int kop_of(xccl_op_t op)
{
    switch (op) {
    case XCCL_OP_MAX:  return K_MAX;
    case XCCL_OP_MIN:  return K_MIN;
    case XCCL_OP_SUM:  return K_SUM;
    case XCCL_OP_PROD: return K_PROD;
    case XCCL_OP_LAND: return K_LAND;
    case XCCL_OP_LOR:  return K_LOR;
    case XCCL_OP_LXOR: return K_LXOR;
    case XCCL_OP_BAND: return K_BAND;
    case XCCL_OP_BOR:  return K_BOR;
    case XCCL_OP_BXOR: return K_BXOR;
    default:           return -1; // AND/OR/XOR/MAXLOC/MINLOC: no kernel
    }
}

// The kernel family for (dtype, op), or NULL.  Coverage follows the
// reference kernels' switch (xccl_cuda_reduce_multi.cu:118-138) widened to
// 8-bit, unsigned and binary16 element types.
const KernelEntry *lookup(xccl_dt_t dt, xccl_op_t op)
{
    const int kop = kop_of(op);
    if (kop < 0) {
        return nullptr;
    }
    bool is_signed = false;
    int  bytes     = 0;
    switch (dt) {
    case XCCL_DT_INT8:   is_signed = true; bytes = 1; break;
    case XCCL_DT_INT16:  is_signed = true; bytes = 2; break;
    case XCCL_DT_INT32:  is_signed = true; bytes = 4; break;
    case XCCL_DT_INT64:  is_signed = true; bytes = 8; break;
    case XCCL_DT_UINT8:  bytes = 1; break;
    case XCCL_DT_UINT16: bytes = 2; break;
    case XCCL_DT_UINT32: bytes = 4; break;
    case XCCL_DT_UINT64: bytes = 8; break;
    case XCCL_DT_FLOAT16: return lookup_fp(kop, 2);
    case XCCL_DT_FLOAT32: return lookup_fp(kop, 4);
    case XCCL_DT_FLOAT64: return lookup_fp(kop, 8);
    default:             return nullptr; // 128-bit integers, unknown
    }
    if (kop >= K_BAND) {
        return lookup_w8(kop, false);
    }
    switch (bytes) {
    case 1:  return lookup_w8(kop, is_signed);
    case 2:  return lookup_w16(kop, is_signed);
    case 4:  return lookup_w32(kop, is_signed);
    default: return lookup_w64(kop, is_signed);
    }
}

struct Plan {
    const void *fn;
    unsigned    grid;
    unsigned    lds_bytes; // dynamic LDS asked for only to bound resident workgroups per CU
    ReduceArgs  args;
};

// LDS per workgroup that lets `resident` workgroups share a compute unit.
// `footprint`: bytes the call touches.  Measured (fp32/fp64/fp16 SUM, 256 MiB
// vectors, rotating destination): 2 sources want every wave slot (7.0 TB/s
// against 6.4 at 16), 3 sources 20 (6.76), 4 to 16 sources 16 (6.6-6.76; 6.2-6.5
// without a cap).  A call whose vectors all fit the 256 MB memory-side cache
// (the integer sweep's 16 Mi-element vectors of 1 and 2 bytes) is served from
// there when its operands were just written, and wants every slot as well
// (int8 SUM, 4 sources: 6.86 TB/s against 6.26 at 16).
unsigned lds_for_resident(uint32_t nsrc, size_t grid, int cus, size_t footprint)
{
    int cap = g_resident.load(std::memory_order_relaxed);
    if (cap == 0) {
        // 8 and more sources want the bound from 8 MiB vectors on (16 sources x 8 MiB: 6.85 TB/s against
        // 6.36 without, 8 x 8 MiB: 6.62 against 6.46), fewer sources only once the call outgrows the cache
        const size_t fits = (size_t)(nsrc >= 8 ? 64 : 192) << 20;
        cap = (nsrc <= 2 || footprint <= fits) ? kNoResidentCap : nsrc == 3 ? 20 : 16;
    }
    if (cap >= kNoResidentCap || grid <= (size_t)cap * (size_t)cus) {
        return 0; // the whole grid is resident at once anyway
    }
    size_t lds = (kLdsPerCu / (size_t)cap) & ~(size_t)511;
    return (unsigned)(lds > kLdsPerGroup ? kLdsPerGroup : lds); // 1 or 2 asked for: 2.5 is the fewest LDS can enforce
}

bool same_plan(const Plan &a, const Plan &b)
{
    return a.fn == b.fn && a.grid == b.grid && a.lds_bytes == b.lds_bytes && a.args.s1 == b.args.s1 && a.args.s2 == b.args.s2 &&
           a.args.dst == b.args.dst && a.args.stride == b.args.stride && a.args.head == b.args.head &&
           a.args.nvec == b.args.nvec && a.args.tail == b.args.tail && a.args.n2 == b.args.n2 &&
           a.args.grid == b.args.grid &&
           a.args.done_flag == b.args.done_flag && a.args.done_count == b.args.done_count &&
           a.args.done_slots == b.args.done_slots &&
           a.args.done_seq == b.args.done_seq;
}

// Bytes to peel so that as many of the buffers as possible start their
// vector body on a 16-byte boundary; ties go to the destination.
size_t pick_head_bytes(const void *s1, const void *s2, const void *dst, size_t stride, uint32_t n2, size_t esize)
{
    unsigned votes[16] = {0};
    votes[(uintptr_t)s1 & 15]++;
    const uint32_t look = n2 < 32 ? n2 : 32;
    for (uint32_t j = 0; j < look; ++j) {
        votes[((uintptr_t)s2 + (size_t)j * stride) & 15]++;
    }
    const unsigned dm = (unsigned)((uintptr_t)dst & 15);
    votes[dm]++;
    unsigned best = 16, best_votes = 0;
    for (unsigned m = 0; m < 16; ++m) {
        if (m % esize != 0 || votes[m] == 0) {
            continue; // cannot be reached by peeling whole elements
        }
        if (votes[m] > best_votes || (votes[m] == best_votes && m == dm)) {
            best       = m;
            best_votes = votes[m];
        }
    }
    return best == 16 ? 0 : (16 - best) % 16;
}

xccl_status_t make_plan(void *s1, void *s2, void *dst, size_t count, size_t size, size_t stride, xccl_dt_t dt,
                        xccl_op_t op, Plan *plan)
{
    const KernelEntry *e = lookup(dt, op);
    if (e == nullptr) {
        return XCCL_ERR_UNSUPPORTED;
    }
    if (s1 == nullptr || s2 == nullptr || dst == nullptr) {
        return XCCL_ERR_INVALID_PARAM;
    }
    if (count > 0xffffffffu || size > ((size_t)1 << 56)) {
        return XCCL_ERR_INVALID_PARAM; // byte counts and vector indices below stay far from wrapping
    }
    read_env_once();
    int cus = 0;
    xccl_status_t st = cu_count(&cus);
    if (st != XCCL_OK) {
        return st;
    }

    const size_t   esize = (size_t)e->elem_size;
    const size_t   elems = size * (xccl_dt_size(dt) / esize); // bitwise ops fold bytes
    const size_t   ve    = 16 / esize;
    const uint32_t n2    = count == 0 ? 1u : (uint32_t)count;
    const uint32_t nsrc  = n2 + 1;

    size_t head = pick_head_bytes(s1, s2, dst, stride, n2, esize) / esize;
    if (head > elems) {
        head = elems;
    }
    ReduceArgs &a = plan->args;
    a.s1     = (const char *)s1 + head * esize; // the kernel works relative to the vector body
    a.s2     = (const char *)s2 + head * esize;
    a.dst    = (char *)dst + head * esize;
    a.stride = stride;
    a.head   = head;
    a.nvec   = (elems - head) / ve;
    a.tail   = (elems - head) % ve;
    a.n2     = n2;
    a.done_seq   = 0;
    a.done_count = nullptr;
    a.done_slots = 0;
    a.done_flag  = nullptr;

    const size_t tile  = (size_t)kBlock;
    const size_t tiles = (a.nvec + tile - 1) / tile;
    const size_t cap   = (size_t)cus * (size_t)g_blocks_per_cu.load(std::memory_order_relaxed);
    size_t       grid  = tiles < cap ? tiles : cap;
    if (grid == 0) {
        grid = 1; // head/tail only
    }
    plan->grid      = (unsigned)grid;
    a.grid          = (uint32_t)grid;
    plan->lds_bytes = lds_for_resident(nsrc, grid, cus, (size_t)(nsrc + 1) * elems * esize);
    plan->fn        = (nsrc >= 4 && grid <= g_burst_max_grid.load(std::memory_order_relaxed)) ? e->fn_burst : e->fn;
    return XCCL_OK;
}

// The k-nomial and scatter-reduce rounds repeat identical calls (same buffers,
// same shape) collective after collective; every thread keeps the plan of its
// last call and skips kernel lookup, alignment vote and grid sizing when the
// next call has the same arguments.
struct PlanKey {
    void     *s1, *s2, *dst;
    size_t    count, size, stride;
    int       dt, op;
    unsigned  epoch;
};

struct PlanCache {
    bool    valid = false;
    PlanKey key;
    Plan    plan;
};

thread_local PlanCache t_plan;

xccl_status_t cached_plan(void *s1, void *s2, void *dst, size_t count, size_t size, size_t stride, xccl_dt_t dt,
                          xccl_op_t op, Plan *plan)
{
    const unsigned epoch = g_shape_epoch.load(std::memory_order_acquire);
    PlanCache     &c     = t_plan;
    if (c.valid && c.key.s1 == s1 && c.key.s2 == s2 && c.key.dst == dst && c.key.count == count && c.key.size == size &&
        c.key.stride == stride && c.key.dt == (int)dt && c.key.op == (int)op && c.key.epoch == epoch) {
        *plan = c.plan;
        return XCCL_OK;
    }
    xccl_status_t st = make_plan(s1, s2, dst, count, size, stride, dt, op, plan);
    if (st == XCCL_OK) {
        c.key   = PlanKey{s1, s2, dst, count, size, stride, (int)dt, (int)op, epoch};
        c.plan  = *plan;
        c.valid = true;
    }
    return st;
}

static_assert(XCCL_ROCM_DONE_COUNT_BYTES == (1 + kDoneShards) * kDoneStride * sizeof(uint32_t), "counter block size");

// ---- single-kernel-node graph cache ---------------------------------------
constexpr int kGraphSlots = 8;

struct GraphSlot {
    bool            live = false;
    Plan            plan;
    hipGraph_t      graph = nullptr;
    hipGraphNode_t  node  = nullptr;
    hipGraphExec_t  exec  = nullptr;
    hipStream_t     last_stream = nullptr; // where the last launch went
    bool            last_stream_valid = false;
    uint64_t        stamp = 0;
};

struct GraphCache {
    std::mutex lock;
    GraphSlot  slot[kGraphSlots];
    uint64_t   clock = 0;
};

GraphCache g_graphs[kMaxDevices];

void fill_node_params(hipKernelNodeParams *p, Plan *plan, void **argv)
{
    argv[0] = &plan->args;
    memset(p, 0, sizeof(*p));
    p->func           = const_cast<void *>(plan->fn);
    p->gridDim        = dim3(plan->grid, 1, 1);
    p->blockDim       = dim3(kBlock, 1, 1);
    p->sharedMemBytes = plan->lds_bytes;
    p->kernelParams   = argv;
    p->extra          = nullptr;
}

void destroy_slot(GraphSlot &s)
{
    if (s.exec) {
        (void)hipGraphExecDestroy(s.exec);
    }
    if (s.graph) {
        (void)hipGraphDestroy(s.graph);
    }
    s = GraphSlot();
}

#define HIP_OR_FAIL(call)                                                                          \
    do {                                                                                           \
        hipError_t e_ = (call);                                                                    \
        if (e_ != hipSuccess) {                                                                    \
            fprintf(stderr, "xccl mc_rocm: %s failed: %s\n", #call, hipGetErrorString(e_));        \
            return XCCL_ERR_NO_MESSAGE;                                                            \
        }                                                                                          \
    } while (0)

uint64_t clock_ns()
{
    timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (uint64_t)ts.tv_sec * 1000000000ull + (uint64_t)ts.tv_nsec;
}

// Launches `plan` as a one-node graph: a slot whose instantiated graph has the
// same arguments is replayed untouched, otherwise the least recently used slot
// is patched.  `ns` (may be NULL) receives the host time of the three steps:
// [0] lock + slot search, [1] building or patching the graph, [2] hipGraphLaunch.
xccl_status_t graph_launch(Plan &plan, hipStream_t stream, uint64_t *ns)
{
    int dev = 0;
    HIP_OR_FAIL(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) {
        return XCCL_ERR_NO_RESOURCE;
    }
    uint64_t                    t = ns ? clock_ns() : 0;
    GraphCache                 &gc = g_graphs[dev];
    std::lock_guard<std::mutex> guard(gc.lock);

    GraphSlot *hit = nullptr, *victim = nullptr;
    for (GraphSlot &s : gc.slot) {
        if (s.live && same_plan(s.plan, plan)) {
            hit = &s;
            break;
        }
    }
    if (hit == nullptr) {
        for (GraphSlot &s : gc.slot) { // a free slot, else the least recently used
            if (!s.live) {
                victim = &s;
                break;
            }
            if (victim == nullptr || s.stamp < victim->stamp) {
                victim = &s;
            }
        }
    }
    if (ns) {
        const uint64_t u = clock_ns();
        ns[0] = u - t;
        t     = u;
    }

    if (hit == nullptr) {
        hipKernelNodeParams np;
        void               *argv[1];
        if (!victim->live) {
            victim->plan = plan;
            fill_node_params(&np, &victim->plan, argv);
            HIP_OR_FAIL(hipGraphCreate(&victim->graph, 0));
            if (hipGraphAddKernelNode(&victim->node, victim->graph, nullptr, 0, &np) != hipSuccess ||
                hipGraphInstantiate(&victim->exec, victim->graph, nullptr, nullptr, 0) != hipSuccess) {
                destroy_slot(*victim);
                (void)hipGetLastError();
                return XCCL_ERR_NO_MESSAGE;
            }
            victim->live = true;
        } else {
            // The executable graph may still be running its previous launch;
            // patch it only once that launch has finished.
            if (victim->last_stream_valid) {
                HIP_OR_FAIL(hipStreamSynchronize(victim->last_stream));
            }
            victim->plan = plan;
            fill_node_params(&np, &victim->plan, argv);
            if (hipGraphExecKernelNodeSetParams(victim->exec, victim->node, &np) != hipSuccess) {
                destroy_slot(*victim);
                (void)hipGetLastError();
                return XCCL_ERR_NO_MESSAGE;
            }
        }
        hit = victim;
    }
    if (ns) {
        const uint64_t u = clock_ns();
        ns[1] = u - t;
        t     = u;
    }
    hit->stamp = ++gc.clock;
    HIP_OR_FAIL(hipGraphLaunch(hit->exec, stream));
    hit->last_stream       = stream;
    hit->last_stream_valid = true;
    if (ns) {
        ns[2] = clock_ns() - t;
    }
    return XCCL_OK;
}

// Completion word of a launch too large to count its own workgroups: a
// one-lane kernel queued right behind it.  Stream order makes it start after
// the reduction has finished and its results are visible system-wide.
__global__ void tail_flag_kernel(uint32_t *flag, uint32_t seq)
{
    __hip_atomic_store(flag, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Polls *flag (host-mapped) from one lane; see xccl_rocm_stream_gate.
__global__ void stream_gate_kernel(int *flag, uint64_t max_ticks)
{
    const uint64_t t0 = wall_clock64();
    while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) == 0) {
        if (wall_clock64() - t0 > max_ticks) {
            __hip_atomic_store(flag, 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            break;
        }
        __builtin_amdgcn_s_sleep(16);
    }
}

} // namespace
} // namespace xccl_rocm

using namespace xccl_rocm;

namespace {

// Plan of a call, or `*nothing` when there is nothing to launch (size == 0 is
// a no-op for a supported pair, reference mem_component.c:129-131).
xccl_status_t prepare(void *s1, void *s2, void *dst, size_t count, size_t size, size_t stride, xccl_dt_t dt,
                      xccl_op_t op, Plan *plan, bool *nothing)
{
    *nothing = size == 0;
    if (size == 0) {
        return lookup(dt, op) ? XCCL_OK : XCCL_ERR_UNSUPPORTED;
    }
    return cached_plan(s1, s2, dst, count, size, stride, dt, op, plan);
}

// Arrival counters for xccl_rocm_reduce_multi_flagged_static: device memory that
// exists from the moment the code object is loaded, so that entry never
// allocates.  In host code the array's name is a stand-in, not a device
// address: the address on each device comes from hipGetSymbolAddress, once per
// device, and only that pointer is ever handed to a kernel.
static __device__ __align__(256) uint32_t scratch[XCCL_ROCM_DONE_COUNT_BYTES / sizeof(uint32_t)];

std::atomic<uint32_t *> g_scratch_ptr[kMaxDevices];
std::mutex              g_scratch_lock;

xccl_status_t static_scratch(uint32_t **out)
{
    int dev = 0;
    HIP_OR_FAIL(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) {
        return XCCL_ERR_NO_RESOURCE;
    }
    uint32_t *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        std::lock_guard<std::mutex> guard(g_scratch_lock);
        p = g_scratch_ptr[dev].load(std::memory_order_relaxed);
        if (p == nullptr) {
            HIP_OR_FAIL(hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch)));
            g_scratch_ptr[dev].store(p, std::memory_order_release);
        }
    }
    *out = p;
    return XCCL_OK;
}

// Clears the arrival counters (a fill kernel, not hipMemsetAsync: callers may be capturing).
__global__ void clear_words_kernel(uint32_t *p, uint32_t n)
{
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) {
        p[i] = 0;
    }
}


// How the host learns that a launch is complete (values of XCCL_ROCM_ROUTE_*):
// one word per workgroup for a handful of workgroups, a word written by the
// last workgroup to arrive for small grids, and for larger ones a one-lane
// kernel queued behind the launch on a HIP stream or the packet's completion
// signal on the component's own queue; else the stream itself.
std::atomic<int> *direct_signal_knob();

int completion_route(const Plan &plan, uint32_t flag_words, bool own_queue, bool want_flag, bool has_signal)
{
    if (!want_flag) {
        return XCCL_ROCM_ROUTE_STREAM;
    }
    const bool     tail_ok   = g_tail_flag.load(std::memory_order_relaxed) != 0;
    const unsigned counted   = own_queue ? g_direct_counted_grid.load(std::memory_order_relaxed)
                               : tail_ok ? g_max_counted_grid.load(std::memory_order_relaxed)
                                         : kMaxFlaggedGrid;
    const unsigned slots_max = flag_words < XCCL_ROCM_FLAG_WORDS ? flag_words : XCCL_ROCM_FLAG_WORDS;
    if (plan.grid <= counted) {
        // a grid of one needs neither counting nor a second word: it stays on the counting path, which then has no atomics
        const bool by_slots = plan.grid > 1 && plan.grid <= slots_max && plan.grid <= g_slot_max_grid.load(std::memory_order_relaxed);
        return by_slots ? XCCL_ROCM_ROUTE_SLOTS : XCCL_ROCM_ROUTE_COUNTED;
    }
    if (own_queue) {
        return has_signal && direct_signal_knob()->load(std::memory_order_relaxed) != 0 ? XCCL_ROCM_ROUTE_SIGNAL
                                                                                         : XCCL_ROCM_ROUTE_STREAM;
    }
    return tail_ok ? XCCL_ROCM_ROUTE_TAIL : XCCL_ROCM_ROUTE_STREAM;
}

// Arms `plan` to write its own completion word (route SLOTS or COUNTED);
// returns how many words the host has to watch.
int arm_completion(Plan &plan, int route, uint32_t *dev_count, uint32_t *dev_flag, uint32_t seq)
{
    const bool by_slots = route == XCCL_ROCM_ROUTE_SLOTS;
    plan.args.done_seq   = seq;
    plan.args.done_count = dev_count;
    plan.args.done_slots = by_slots ? plan.grid : 0;
    plan.args.done_flag  = dev_flag;
    return by_slots ? (int)plan.grid : 1;
}

// ---- the component's own dispatch queues ------------------------------------
// A blocking reduction that completes through its own completion word needs
// nothing of a HIP stream: no event, no ordering against other work.  Such
// launches go out as AQL packets on a user-mode queue the component creates
// through the HSA runtime (the layer HIP itself sits on): the host's part of a
// launch shrinks from ~2.6 us inside hipLaunchKernel, with its locks and pools,
// to writing 64 bytes and ringing a doorbell.  The kernels are the same code,
// loaded a second time from the bare code objects embedded in this library
// (kernel_images.S); they read no implicit launch arguments, so the kernel
// argument block is ReduceArgs and nothing else.  Packets carry the barrier
// bit (launches of one queue run in order) and agent-scope acquire and release
// fences, which is what a kernel launched on a HIP stream gets; the result
// stores are write-through and waited for by the kernel itself.
//   Two queues per device, for the first two of the component's four thread
// slots, each created when a thread of the slot first calls, behind that
// slot's HIP stream; threads of the other slots keep to their HIP streams.
// Measured, blocking call, 4 sources x 1 KiB, p50 / p99 in us: one thread 5.4 /
// 5.7; two threads on a queue each 5.6-6.0 / 6.8-8.4; four threads on a queue
// each 9.5 / 30 (twice, on different boxes), two of them on HIP streams instead
// 7.4 / 11.2, all four on HIP streams 7.2 / 13.4; four threads sharing one queue
// 13.3 / 13.6 (the packet processor takes ~3 us per packet of a queue, fences
// included, one after the other).
extern "C" {
extern const unsigned char *const xccl_rocm_kernel_image_begin[5];
extern const unsigned char *const xccl_rocm_kernel_image_end[5];
}

constexpr int      kMaxDirectQueues = 4; // one per thread slot at most
constexpr int      kDefaultDirectQueues = 2;
constexpr uint32_t kDirectPackets = 256; // queue size; a blocking caller has one launch in flight
constexpr size_t   kKernargSlot   = 128; // >= sizeof(ReduceArgs), one cache line pair per packet
// Twice as many argument slots as packets: a packet is written once the queue has *consumed* the one 256
// before it, which may still be running; with 512 slots an argument block is rewritten only after the packet
// 256 behind its last user has been consumed, and the barrier bit makes that wait for everything before it.
constexpr uint32_t kKernargSlots  = 2 * kDirectPackets;
static_assert(sizeof(ReduceArgs) <= kKernargSlot, "kernel argument slot");
static_assert(XCCL_ROCM_KERNARG_BYTES == kKernargSlot, "kernel argument block a caller brings");

struct DirectKernel {
    uint64_t object = 0; // kernel descriptor address
    uint32_t group  = 0; // static LDS
};

struct DirectQueue {
    hsa_queue_t *q       = nullptr;
    char        *kernarg = nullptr; // kKernargSlots slots, pinned host memory
};

struct DirectDevice {
    std::atomic<int>                              state{0}; // 0 untried, 1 usable, -1 unavailable
    std::atomic<unsigned>                         generation{0}; // bumped when the executable is destroyed
    std::mutex                                    lock;
    hsa_agent_t                                   agent{};
    hsa_executable_t                              exe{};
    hsa_code_object_reader_t                      reader[5]{};
    int                                           readers = 0;
    bool                                          hsa_up  = false;
    std::unordered_map<const void *, DirectKernel> kernels; // by HIP function pointer
    DirectQueue                                   queue[kMaxDirectQueues];
    std::vector<hsa_signal_t>                     signals; // completion signals handed out, destroyed with the queues
};

DirectDevice          g_direct[kMaxDevices];
std::atomic<int>      g_direct_enabled{-1}; // -1: environment not read yet
std::atomic<int>      g_direct_failed{0};   // a queue reported an error: launches on it may never complete
std::atomic<uint64_t> g_direct_launches{0};

// How the component's own queues are used (environment, read with XCCL_MC_ROCM_DIRECT_QUEUE; setters below):
//   g_direct_acquire  scope of the acquire fence in front of a launch: agent (what HIP gives a kernel that
//                     follows other kernels) or system (XCCL_MC_ROCM_DIRECT_ACQUIRE=system)
//   g_direct_queues   queues per device, one per thread slot from slot 0 up (XCCL_MC_ROCM_DIRECT_QUEUES, 1..4)
//   g_direct_share    1: thread slots beyond the last queue share the queues round-robin instead of keeping to
//                     their HIP streams (XCCL_MC_ROCM_DIRECT_SHARE)
//   g_direct_barrier  0: a blocking call's packet does not carry the barrier bit, i.e. does not wait for other
//                     threads' launches on the same queue (XCCL_MC_ROCM_DIRECT_BARRIER)
//   g_direct_signal   1: launches too large to count their own workgroups stay on the own queue and complete
//                     through a completion signal on their packet (XCCL_MC_ROCM_DIRECT_SIGNAL)
std::atomic<uint32_t> g_direct_acquire{HSA_FENCE_SCOPE_AGENT};
std::atomic<int>      g_direct_queues{kDefaultDirectQueues};
std::atomic<int>      g_direct_share{1};
std::atomic<int>      g_direct_barrier{0};
std::atomic<int>      g_direct_signal{0};

std::atomic<int> *direct_signal_knob()
{
    return &g_direct_signal;
}

bool direct_enabled()
{
    int on = g_direct_enabled.load(std::memory_order_acquire);
    if (on < 0) {
        const char *e = getenv("XCCL_MC_ROCM_DIRECT_QUEUE");
        const char *a = getenv("XCCL_MC_ROCM_DIRECT_ACQUIRE");
        const char *n = getenv("XCCL_MC_ROCM_DIRECT_QUEUES");
        const char *h = getenv("XCCL_MC_ROCM_DIRECT_SHARE");
        const char *b = getenv("XCCL_MC_ROCM_DIRECT_BARRIER");
        const char *g = getenv("XCCL_MC_ROCM_DIRECT_SIGNAL");
        if (a != nullptr) {
            g_direct_acquire.store(strcmp(a, "system") == 0 ? HSA_FENCE_SCOPE_SYSTEM : HSA_FENCE_SCOPE_AGENT,
                                   std::memory_order_release);
        }
        if (n != nullptr && atoi(n) >= 1 && atoi(n) <= kMaxDirectQueues) {
            g_direct_queues.store(atoi(n), std::memory_order_release);
        }
        if (h != nullptr) {
            g_direct_share.store(atoi(h) != 0, std::memory_order_release);
        }
        if (b != nullptr) {
            g_direct_barrier.store(atoi(b) != 0, std::memory_order_release);
        }
        if (g != nullptr) {
            g_direct_signal.store(atoi(g) != 0, std::memory_order_release);
        }
        on = (e == nullptr || atoi(e) != 0) ? 1 : 0;
        g_direct_enabled.store(on, std::memory_order_release);
    }
    return on != 0;
}

#define HSA_OR_GIVE_UP(call)                                                                               \
    do {                                                                                                   \
        hsa_status_t s_ = (call);                                                                          \
        if (s_ != HSA_STATUS_SUCCESS) {                                                                    \
            const char *m_ = nullptr;                                                                      \
            (void)hsa_status_string(s_, &m_);                                                              \
            fprintf(stderr, "xccl mc_rocm: %s failed (%s); reductions keep to the HIP stream\n", #call,    \
                    m_ ? m_ : "unknown status");                                                           \
            return false;                                                                                  \
        }                                                                                                  \
    } while (0)

struct AgentSearch {
    uint32_t    bdf;    // bus << 8 | device << 3 (function ignored)
    uint32_t    domain;
    hsa_agent_t found;
    bool        ok;
};

hsa_status_t match_agent(hsa_agent_t agent, void *data)
{
    AgentSearch      *want = static_cast<AgentSearch *>(data);
    hsa_device_type_t type;
    uint32_t          bdf = 0, domain = 0;
    if (hsa_agent_get_info(agent, HSA_AGENT_INFO_DEVICE, &type) != HSA_STATUS_SUCCESS || type != HSA_DEVICE_TYPE_GPU) {
        return HSA_STATUS_SUCCESS;
    }
    if (hsa_agent_get_info(agent, (hsa_agent_info_t)HSA_AMD_AGENT_INFO_BDFID, &bdf) != HSA_STATUS_SUCCESS ||
        hsa_agent_get_info(agent, (hsa_agent_info_t)HSA_AMD_AGENT_INFO_DOMAIN, &domain) != HSA_STATUS_SUCCESS) {
        return HSA_STATUS_SUCCESS;
    }
    if ((bdf & 0xfff8u) == want->bdf && domain == want->domain) {
        want->found = agent;
        want->ok    = true;
        return HSA_STATUS_INFO_BREAK;
    }
    return HSA_STATUS_SUCCESS;
}

void on_queue_error(hsa_status_t status, hsa_queue_t *, void *)
{
    const char *m = nullptr;
    (void)hsa_status_string(status, &m);
    fprintf(stderr, "xccl mc_rocm: the component's dispatch queue reported an error: %s\n", m ? m : "unknown status");
    g_direct_failed.store(1, std::memory_order_release);
}

// Finds the HSA agent of HIP device `dev` (by PCI address) and loads the
// embedded code objects for it.  Caller holds dd.lock.
bool direct_setup(DirectDevice &dd, int dev)
{
    int bus = 0, device = 0, domain = 0;
    if (hipDeviceGetAttribute(&bus, hipDeviceAttributePciBusId, dev) != hipSuccess ||
        hipDeviceGetAttribute(&device, hipDeviceAttributePciDeviceId, dev) != hipSuccess ||
        hipDeviceGetAttribute(&domain, hipDeviceAttributePciDomainID, dev) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    HSA_OR_GIVE_UP(hsa_init());
    dd.hsa_up = true;
    AgentSearch want{(uint32_t)((bus & 0xff) << 8 | (device & 0x1f) << 3), (uint32_t)domain, {}, false};
    hsa_status_t it = hsa_iterate_agents(match_agent, &want);
    if ((it != HSA_STATUS_SUCCESS && it != HSA_STATUS_INFO_BREAK) || !want.ok) {
        fprintf(stderr, "xccl mc_rocm: no HSA agent at PCI %04x:%02x:%02x; reductions keep to the HIP stream\n", domain, bus,
                device);
        return false;
    }
    dd.agent = want.found;
    HSA_OR_GIVE_UP(hsa_executable_create_alt(HSA_PROFILE_FULL, HSA_DEFAULT_FLOAT_ROUNDING_MODE_DEFAULT, nullptr, &dd.exe));
    for (int i = 0; i < 5; ++i) {
        const size_t bytes = (size_t)(xccl_rocm_kernel_image_end[i] - xccl_rocm_kernel_image_begin[i]);
        HSA_OR_GIVE_UP(hsa_code_object_reader_create_from_memory(xccl_rocm_kernel_image_begin[i], bytes, &dd.reader[i]));
        dd.readers = i + 1;
        HSA_OR_GIVE_UP(hsa_executable_load_agent_code_object(dd.exe, dd.agent, dd.reader[i], nullptr, nullptr));
    }
    HSA_OR_GIVE_UP(hsa_executable_freeze(dd.exe, nullptr));
    return true;
}

// Kernel descriptor of the HIP kernel `fn` in the component's own executable.
bool direct_kernel(DirectDevice &dd, const void *fn, DirectKernel *out)
{
    thread_local const void  *last_fn = nullptr;
    thread_local DirectKernel last;
    thread_local const DirectDevice *last_dd = nullptr;
    thread_local unsigned            last_gen = 0;
    const unsigned                   gen      = dd.generation.load(std::memory_order_acquire);
    if (fn == last_fn && last_dd == &dd && last_gen == gen) {
        *out = last;
        return true;
    }
    std::lock_guard<std::mutex> guard(dd.lock);
    auto                        it = dd.kernels.find(fn);
    if (it == dd.kernels.end()) {
        const char *name = hipKernelNameRefByPtr(fn, nullptr);
        if (name == nullptr) {
            return false;
        }
        const std::string       symbol = std::string(name) + ".kd";
        hsa_executable_symbol_t sym;
        uint32_t                kernarg = 0, priv = 0;
        DirectKernel            k;
        HSA_OR_GIVE_UP(hsa_executable_get_symbol_by_name(dd.exe, symbol.c_str(), &dd.agent, &sym));
        HSA_OR_GIVE_UP(hsa_executable_symbol_get_info(sym, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_OBJECT, &k.object));
        HSA_OR_GIVE_UP(hsa_executable_symbol_get_info(sym, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_KERNARG_SEGMENT_SIZE, &kernarg));
        HSA_OR_GIVE_UP(hsa_executable_symbol_get_info(sym, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_GROUP_SEGMENT_SIZE, &k.group));
        HSA_OR_GIVE_UP(hsa_executable_symbol_get_info(sym, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_PRIVATE_SEGMENT_SIZE, &priv));
        if (kernarg != sizeof(ReduceArgs) || priv != 0 || k.object == 0) {
            // implicit launch arguments or scratch memory would need more than this path sets up
            fprintf(stderr, "xccl mc_rocm: kernel %s has %u argument bytes and %u scratch bytes, expected %zu and 0\n", name,
                    kernarg, priv, sizeof(ReduceArgs));
            return false;
        }
        it = dd.kernels.emplace(fn, k).first;
    }
    *out     = it->second;
    last     = it->second;
    last_fn  = fn;
    last_dd  = &dd;
    last_gen = gen;
    return true;
}

bool direct_queue(DirectDevice &dd, int slot, DirectQueue **out)
{
    DirectQueue &dq = dd.queue[slot];
    if (__atomic_load_n(&dq.q, __ATOMIC_ACQUIRE) == nullptr) {
        std::lock_guard<std::mutex> guard(dd.lock);
        if (dq.q == nullptr) {
            char *ring = nullptr;
            if (hipHostMalloc((void **)&ring, kKernargSlots * kKernargSlot, hipHostMallocDefault) != hipSuccess) {
                (void)hipGetLastError();
                return false;
            }
            memset(ring, 0, kKernargSlots * kKernargSlot);
            hsa_queue_t *q = nullptr;
            hsa_status_t st = hsa_queue_create(dd.agent, kDirectPackets, HSA_QUEUE_TYPE_MULTI, on_queue_error, nullptr,
                                               UINT32_MAX, UINT32_MAX, &q);
            if (st != HSA_STATUS_SUCCESS || q == nullptr || q->size != kDirectPackets) {
                if (q != nullptr) {
                    (void)hsa_queue_destroy(q);
                }
                (void)hipHostFree(ring);
                fprintf(stderr, "xccl mc_rocm: no dispatch queue of its own for the component; reductions keep to the HIP "
                                "stream\n");
                return false;
            }
            dq.kernarg = ring;
            __atomic_store_n(&dq.q, q, __ATOMIC_RELEASE);
        }
    }
    *out = &dq;
    return true;
}

// The current device's queues and code, set up on first use; NULL when the
// path is off or could not be set up.
DirectDevice *direct_device()
{
    if (!direct_enabled() || g_direct_failed.load(std::memory_order_acquire) != 0) {
        return nullptr;
    }
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return nullptr;
    }
    DirectDevice &dd    = g_direct[dev];
    int           state = dd.state.load(std::memory_order_acquire);
    if (state == 0) {
        std::lock_guard<std::mutex> guard(dd.lock);
        state = dd.state.load(std::memory_order_relaxed);
        if (state == 0) {
            state = direct_setup(dd, dev) ? 1 : -1;
            dd.state.store(state, std::memory_order_release);
        }
    }
    return state == 1 ? &dd : nullptr;
}

// A completion signal for launches of the current device's queues (destroyed
// with the queues).  Nothing waits on it through the runtime -- the host reads
// its value -- so it needs no interrupt.
bool direct_signal_create(DirectDevice &dd, uint64_t *handle)
{
    std::lock_guard<std::mutex> guard(dd.lock);
    hsa_signal_t                sig{};
    if (hsa_amd_signal_create(0, 0, nullptr, HSA_AMD_SIGNAL_AMD_GPU_ONLY, &sig) != HSA_STATUS_SUCCESS || sig.handle == 0) {
        return false;
    }
    dd.signals.push_back(sig);
    *handle = sig.handle;
    return true;
}

// Puts `plan` on queue `slot` of the current device.  `signal` != 0: the packet
// processor sets that signal to 0 when the launch is complete (the caller set
// nothing: it is armed here).  `ordered`: the launch waits for everything
// queued before it.  Anything but XCCL_OK: nothing was enqueued and the caller
// launches on a HIP stream instead.
xccl_status_t direct_launch(DirectDevice &dd, int slot, const Plan &plan, uint64_t signal, bool ordered, void *kernarg)
{
    if (slot < 0 || slot >= kMaxDirectQueues) {
        return XCCL_ERR_NO_RESOURCE;
    }
    DirectKernel k;
    DirectQueue *dq = nullptr;
    if (!direct_kernel(dd, plan.fn, &k) || !direct_queue(dd, slot, &dq)) {
        dd.state.store(-1, std::memory_order_release); // do not try again on every call
        return XCCL_ERR_NO_RESOURCE;
    }
    if ((size_t)k.group + plan.lds_bytes > kLdsPerGroup) {
        return XCCL_ERR_NO_RESOURCE;
    }

    hsa_queue_t   *q   = dq->q;
    const uint64_t idx = hsa_queue_add_write_index_scacq_screl(q, 1);
    while (idx - hsa_queue_load_read_index_scacquire(q) >= q->size) {
        // queue full: kDirectPackets launches waiting to start; wait for the oldest
        if (g_direct_failed.load(std::memory_order_acquire) != 0) {
            return XCCL_ERR_NO_RESOURCE; // the queue is dead; the reserved packet stays invalid
        }
    }
    // the caller's own argument block (its until the launch is complete), else the queue's ring
    char *args = kernarg != nullptr ? static_cast<char *>(kernarg) : dq->kernarg + (idx & (kKernargSlots - 1)) * kKernargSlot;
    memcpy(args, &plan.args, sizeof(ReduceArgs));

    hsa_kernel_dispatch_packet_t *p = static_cast<hsa_kernel_dispatch_packet_t *>(q->base_address) + (idx & (q->size - 1));
    p->workgroup_size_x     = kBlock;
    p->workgroup_size_y     = 1;
    p->workgroup_size_z     = 1;
    p->reserved0            = 0;
    p->grid_size_x          = plan.grid * (uint32_t)kBlock; // in work-items
    p->grid_size_y          = 1;
    p->grid_size_z          = 1;
    p->private_segment_size = 0;
    p->group_segment_size   = k.group + plan.lds_bytes;
    p->kernel_object        = k.object;
    p->kernarg_address      = args;
    p->reserved2            = 0;
    p->completion_signal.handle = signal; // 0: completion is the kernel's own word
    if (signal != 0) {
        hsa_signal_store_relaxed(hsa_signal_t{signal}, 1);
    }
    const uint32_t header = (uint32_t)HSA_PACKET_TYPE_KERNEL_DISPATCH << HSA_PACKET_HEADER_TYPE |
                            (ordered ? 1u : 0u) << HSA_PACKET_HEADER_BARRIER |
                            g_direct_acquire.load(std::memory_order_relaxed) << HSA_PACKET_HEADER_SCACQUIRE_FENCE_SCOPE |
                            (uint32_t)HSA_FENCE_SCOPE_AGENT << HSA_PACKET_HEADER_SCRELEASE_FENCE_SCOPE;
    const uint32_t setup  = 1u << HSA_KERNEL_DISPATCH_PACKET_SETUP_DIMENSIONS;
    // header and setup share the packet's first 32-bit word: one release store makes the packet valid
    __atomic_store_n(reinterpret_cast<uint32_t *>(p), header | setup << 16, __ATOMIC_RELEASE);
    hsa_signal_store_screlease(q->doorbell_signal, (hsa_signal_value_t)idx);
    g_direct_launches.fetch_add(1, std::memory_order_relaxed);
    return XCCL_OK;
}

// Waits until everything queued on `q` has completed: a barrier packet with a
// completion signal goes in behind it (a stream-ordered launch whose event
// nobody waited for may still be queued or running when the component closes).
// Bounded: gives up after `limit_ns`, or when the queue has reported an error.
void direct_drain(hsa_queue_t *q, uint64_t limit_ns)
{
    hsa_signal_t done{};
    if (g_direct_failed.load(std::memory_order_acquire) != 0 ||
        hsa_amd_signal_create(1, 0, nullptr, HSA_AMD_SIGNAL_AMD_GPU_ONLY, &done) != HSA_STATUS_SUCCESS) {
        return;
    }
    const uint64_t t0  = clock_ns();
    const uint64_t idx = hsa_queue_add_write_index_scacq_screl(q, 1);
    bool           room = true;
    while (idx - hsa_queue_load_read_index_scacquire(q) >= q->size) {
        if (g_direct_failed.load(std::memory_order_acquire) != 0 || clock_ns() - t0 > limit_ns) {
            room = false; // the reserved packet stays invalid; the queue is about to be destroyed anyway
            break;
        }
    }
    if (room) {
        hsa_barrier_and_packet_t *b = static_cast<hsa_barrier_and_packet_t *>(q->base_address) + (idx & (q->size - 1));
        memset(reinterpret_cast<char *>(b) + 4, 0, sizeof(*b) - 4);
        b->completion_signal = done;
        const uint32_t header = (uint32_t)HSA_PACKET_TYPE_BARRIER_AND << HSA_PACKET_HEADER_TYPE |
                                1u << HSA_PACKET_HEADER_BARRIER |
                                (uint32_t)HSA_FENCE_SCOPE_AGENT << HSA_PACKET_HEADER_SCACQUIRE_FENCE_SCOPE |
                                (uint32_t)HSA_FENCE_SCOPE_AGENT << HSA_PACKET_HEADER_SCRELEASE_FENCE_SCOPE;
        __atomic_store_n(reinterpret_cast<uint32_t *>(b), header, __ATOMIC_RELEASE);
        hsa_signal_store_screlease(q->doorbell_signal, (hsa_signal_value_t)idx);
        while (hsa_signal_load_scacquire(done) != 0) {
            if (g_direct_failed.load(std::memory_order_acquire) != 0 || clock_ns() - t0 > limit_ns) {
                fprintf(stderr, "xccl mc_rocm: the component's dispatch queue did not drain; destroying it anyway\n");
                break;
            }
        }
    }
    (void)hsa_signal_destroy(done);
}

// Releases the queues and the executable of one device, after everything
// queued there has completed.
void direct_destroy(DirectDevice &dd)
{
    std::lock_guard<std::mutex> guard(dd.lock);
    for (DirectQueue &dq : dd.queue) {
        if (dq.q != nullptr) {
            direct_drain(dq.q, 10000000000ull);
            (void)hsa_queue_destroy(dq.q);
            dq.q = nullptr;
        }
        if (dq.kernarg != nullptr) {
            (void)hipHostFree(dq.kernarg);
            dq.kernarg = nullptr;
        }
    }
    for (hsa_signal_t sig : dd.signals) {
        (void)hsa_signal_destroy(sig);
    }
    dd.signals.clear();
    dd.kernels.clear();
    dd.generation.fetch_add(1, std::memory_order_release); // kernel descriptors cached by the threads are stale now
    if (dd.exe.handle != 0) {
        (void)hsa_executable_destroy(dd.exe);
        dd.exe.handle = 0;
    }
    for (int i = 0; i < dd.readers; ++i) {
        (void)hsa_code_object_reader_destroy(dd.reader[i]);
    }
    dd.readers = 0;
    if (dd.hsa_up) {
        (void)hsa_shut_down();
        dd.hsa_up = false;
    }
    dd.state.store(0, std::memory_order_release);
}

} // namespace

extern "C" {

xccl_status_t xccl_rocm_prepare_device(void)
{
    int           cus = 0;
    uint32_t     *p   = nullptr;
    xccl_status_t st  = cu_count(&cus);
    if (st == XCCL_OK) {
        st = static_scratch(&p);
    }
    if (st == XCCL_OK) {
        // the component's own dispatch queue: loading the code and creating a queue takes milliseconds, which
        // belong here and not into the first small reduction; failure leaves the stream path.  Only the first
        // calling thread's queue: the others are created when a thread of their slot first calls.  (The
        // device serves the queue created last fastest: an empty kernel's completion word is seen 4.6 us
        // after the doorbell on the newest of up to 12 open queues, 4.8-5.5 us on the older ones.)
        DirectDevice *dd = direct_device();
        DirectQueue  *dq = nullptr;
        if (dd != nullptr && !direct_queue(*dd, 0, &dq)) {
            dd->state.store(-1, std::memory_order_release);
        }
    }
    return st;
}

xccl_status_t xccl_rocm_reduce_supported(xccl_dt_t dtype, xccl_op_t op)
{
    return lookup(dtype, op) ? XCCL_OK : XCCL_ERR_UNSUPPORTED;
}

xccl_status_t xccl_rocm_reduce_multi_impl(void *sbuf1, void *sbuf2, void *rbuf, size_t count, size_t size,
                                          size_t stride, xccl_dt_t dtype, xccl_op_t op, void *hip_stream)
{
    return xccl_rocm_reduce_multi_flagged(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, hip_stream, nullptr,
                                          nullptr, 0, nullptr);
}

xccl_status_t xccl_rocm_reduce_multi_flagged(void *sbuf1, void *sbuf2, void *rbuf, size_t count, size_t size,
                                             size_t stride, xccl_dt_t dtype, xccl_op_t op, void *hip_stream,
                                             uint32_t *dev_count, uint32_t *dev_flag, uint32_t seq, int *flagged)
{
    return xccl_rocm_reduce_multi_slots(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, hip_stream, dev_count,
                                        dev_flag, 1, seq, flagged);
}

xccl_status_t xccl_rocm_reduce_multi_direct(void *sbuf1, void *sbuf2, void *rbuf, size_t count, size_t size,
                                            size_t stride, xccl_dt_t dtype, xccl_op_t op, int queue_slot,
                                            uint32_t *dev_count, uint32_t *dev_flag, uint32_t flag_words, uint32_t seq,
                                            uint64_t *signal, void *kernarg, int blocking, int *flagged)
{
    if (flagged == nullptr || dev_count == nullptr || dev_flag == nullptr) {
        return XCCL_ERR_INVALID_PARAM;
    }
    *flagged = 0;
    Plan          plan;
    bool          nothing = false;
    xccl_status_t st      = prepare(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, &plan, &nothing);
    if (st != XCCL_OK || nothing) {
        return st;
    }
    DirectDevice *dd = direct_device();
    if (dd == nullptr || queue_slot < 0) {
        return XCCL_OK; // the caller takes the stream path
    }
    const int queues = g_direct_queues.load(std::memory_order_relaxed);
    if (queue_slot >= queues) {
        if (g_direct_share.load(std::memory_order_relaxed) == 0) {
            return XCCL_OK; // this thread slot keeps to its HIP stream
        }
        queue_slot %= queues;
    }
    // A blocking caller has waited for its own earlier launches: its packet need not wait for other threads'.
    // Such a packet may still be running when the queue's argument ring comes round again, so it must bring
    // an argument block of its own.
    const bool ordered  = blocking == 0 || kernarg == nullptr || g_direct_barrier.load(std::memory_order_relaxed) != 0;
    const int route = completion_route(plan, flag_words, true, true, signal != nullptr);
    if (route == XCCL_ROCM_ROUTE_STREAM) {
        return XCCL_OK; // too many workgroups to count themselves: the launch completes through the stream
    }
    if (route == XCCL_ROCM_ROUTE_SIGNAL) {
        if (*signal == 0 && !direct_signal_create(*dd, signal)) {
            return XCCL_OK;
        }
        if (direct_launch(*dd, queue_slot, plan, *signal, ordered, kernarg) == XCCL_OK) {
            *flagged = -1;
        }
        return XCCL_OK;
    }
    const int words = arm_completion(plan, route, dev_count, dev_flag, seq);
    if (direct_launch(*dd, queue_slot, plan, 0, ordered, kernarg) != XCCL_OK) {
        return XCCL_OK; // not launched: the caller takes the stream path
    }
    *flagged = words;
    return XCCL_OK;
}

int xccl_rocm_direct_signal_done(uint64_t signal)
{
    return hsa_signal_load_scacquire(hsa_signal_t{signal}) == 0;
}

void xccl_rocm_set_counted_grid(int on_stream, int on_own_queue)
{
    read_env_once();
    if (on_stream >= 0 && (unsigned)on_stream <= kMaxCountedGridKnob) {
        g_max_counted_grid.store((unsigned)on_stream, std::memory_order_release);
    }
    if (on_own_queue >= 0 && (unsigned)on_own_queue <= kMaxCountedGridKnob) {
        g_direct_counted_grid.store((unsigned)on_own_queue, std::memory_order_release);
    }
    g_shape_epoch.fetch_add(1, std::memory_order_release);
}

void xccl_rocm_set_direct_options(int acquire_system, int queues, int share, int barrier, int signal)
{
    (void)direct_enabled(); // environment first, so that it does not overwrite these later
    if (acquire_system >= 0) {
        g_direct_acquire.store(acquire_system ? HSA_FENCE_SCOPE_SYSTEM : HSA_FENCE_SCOPE_AGENT, std::memory_order_release);
    }
    if (queues >= 1 && queues <= kMaxDirectQueues) {
        g_direct_queues.store(queues, std::memory_order_release);
    }
    if (share >= 0) {
        g_direct_share.store(share != 0, std::memory_order_release);
    }
    if (barrier >= 0) {
        g_direct_barrier.store(barrier != 0, std::memory_order_release);
    }
    if (signal >= 0) {
        g_direct_signal.store(signal != 0, std::memory_order_release);
    }
}

uint64_t xccl_rocm_direct_launch_count(void)
{
    return g_direct_launches.load(std::memory_order_relaxed);
}

int xccl_rocm_direct_queue_failed(void)
{
    return g_direct_failed.load(std::memory_order_acquire);
}

void xccl_rocm_set_direct_queue(int on)
{
    read_env_once();
    g_direct_enabled.store(on != 0 ? 1 : 0, std::memory_order_release);
}

void xccl_rocm_direct_queue_destroy(void)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return;
    }
    direct_destroy(g_direct[dev]);
}

xccl_status_t xccl_rocm_reduce_multi_slots(void *sbuf1, void *sbuf2, void *rbuf, size_t count, size_t size,
                                           size_t stride, xccl_dt_t dtype, xccl_op_t op, void *hip_stream,
                                           uint32_t *dev_count, uint32_t *dev_flag, uint32_t flag_words, uint32_t seq,
                                           int *flagged)
{
    if (flagged) {
        *flagged = 0;
    }
    Plan          plan;
    bool          nothing = false;
    xccl_status_t st      = prepare(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, &plan, &nothing);
    if (st != XCCL_OK || nothing) {
        return st;
    }
    // Who writes the completion word: the launch itself, counting its workgroups (cheapest for small
    // grids), or a one-lane kernel queued behind it (cheaper from a few thousand workgroups on).  The
    // second relies on every result store of the reduction being a write-through store: those are in
    // memory when the reduction kernel ends, and stream order starts the one-lane kernel after that.
    const bool want_flag = dev_count != nullptr && dev_flag != nullptr && flagged != nullptr;
    const int  route     = completion_route(plan, flag_words, false, want_flag, false);
    const bool in_kernel = route == XCCL_ROCM_ROUTE_SLOTS || route == XCCL_ROCM_ROUTE_COUNTED;
    const int  words     = in_kernel ? arm_completion(plan, route, dev_count, dev_flag, seq) : 0;
    void *argv[1] = {&plan.args};
    HIP_OR_FAIL(hipLaunchKernel(plan.fn, dim3(plan.grid, 1, 1), dim3(kBlock, 1, 1), argv, plan.lds_bytes,
                                (hipStream_t)hip_stream));
    if (in_kernel) {
        *flagged = words;
    } else if (route == XCCL_ROCM_ROUTE_TAIL) {
        hipLaunchKernelGGL(tail_flag_kernel, dim3(1), dim3(1), 0, (hipStream_t)hip_stream, dev_flag, seq);
        if (hipGetLastError() == hipSuccess) {
            *flagged = 1; // otherwise the caller waits for the stream, which still works
        }
    }
    return XCCL_OK;
}

xccl_status_t xccl_rocm_reduce_multi_flagged_static(void *sbuf1, void *sbuf2, void *rbuf, size_t count, size_t size,
                                                    size_t stride, xccl_dt_t dtype, xccl_op_t op, void *hip_stream,
                                                    uint32_t *dev_flag, uint32_t seq)
{
    if (dev_flag == nullptr) {
        return XCCL_ERR_INVALID_PARAM;
    }
    Plan          plan;
    bool          nothing = false;
    xccl_status_t st      = prepare(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, &plan, &nothing);
    if (st != XCCL_OK) {
        return st;
    }
    if (nothing) {
        // nothing to reduce, but the caller polls the word: a one-lane kernel stores it, in stream order
        hipLaunchKernelGGL(tail_flag_kernel, dim3(1), dim3(1), 0, (hipStream_t)hip_stream, dev_flag, seq);
        HIP_OR_FAIL(hipGetLastError());
        return XCCL_OK;
    }
    if (plan.grid > kMaxFlaggedGrid) {
        fprintf(stderr,
                "xccl mc_rocm: xccl_rocm_reduce_multi_flagged_static takes at most %u KiB per vector (%u workgroups); "
                "this call needs %u workgroups\n",
                kMaxFlaggedGrid, kMaxFlaggedGrid, plan.grid);
        return XCCL_ERR_INVALID_PARAM;
    }
    uint32_t *counters = nullptr;
    st = static_scratch(&counters);
    if (st != XCCL_OK) {
        return st;
    }
    // The array keeps what the last call on this device left in it; a launch that
    // ran to its end left zeros, one that did not may have left anything.
    hipLaunchKernelGGL(clear_words_kernel, dim3(1), dim3(256), 0, (hipStream_t)hip_stream, counters,
                       (uint32_t)(XCCL_ROCM_DONE_COUNT_BYTES / sizeof(uint32_t)));
    HIP_OR_FAIL(hipGetLastError());
    plan.args.done_seq   = seq;
    plan.args.done_count = counters;
    plan.args.done_flag  = dev_flag;
    void *argv[1] = {&plan.args};
    HIP_OR_FAIL(hipLaunchKernel(plan.fn, dim3(plan.grid, 1, 1), dim3(kBlock, 1, 1), argv, plan.lds_bytes,
                                (hipStream_t)hip_stream));
    return XCCL_OK;
}

xccl_status_t xccl_rocm_reduce_impl(void *sbuf1, void *sbuf2, void *target, size_t count, xccl_dt_t dtype,
                                    xccl_op_t op, void *hip_stream)
{
    return xccl_rocm_reduce_multi_impl(sbuf1, sbuf2, target, 1, count, 0, dtype, op, hip_stream);
}

xccl_status_t xccl_rocm_reduce_multi_graph(void *sbuf1, void *sbuf2, void *rbuf, size_t count, size_t size,
                                           size_t stride, xccl_dt_t dtype, xccl_op_t op, void *hip_stream)
{
    return xccl_rocm_reduce_multi_graph_flagged(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, hip_stream, nullptr,
                                                nullptr, 0, nullptr, nullptr);
}

xccl_status_t xccl_rocm_reduce_multi_graph_flagged(void *sbuf1, void *sbuf2, void *rbuf, size_t count, size_t size,
                                                   size_t stride, xccl_dt_t dtype, xccl_op_t op, void *hip_stream,
                                                   uint32_t *dev_count, uint32_t *dev_flag, uint32_t seq,
                                                   int *flagged, uint64_t *ns_parts)
{
    if (flagged) {
        *flagged = 0;
    }
    const uint64_t t0 = ns_parts ? clock_ns() : 0;
    Plan           plan;
    bool           nothing = false;
    xccl_status_t  st      = prepare(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, &plan, &nothing);
    if (st != XCCL_OK || nothing) {
        return st;
    }
    if (dev_count != nullptr && dev_flag != nullptr && flagged != nullptr && plan.grid <= kMaxFlaggedGrid) {
        plan.args.done_seq   = seq;
        plan.args.done_count = dev_count;
        plan.args.done_flag  = dev_flag;
        *flagged             = 1;
    }
    if (ns_parts) {
        ns_parts[0] = clock_ns() - t0; // planning
    }
    st = graph_launch(plan, (hipStream_t)hip_stream, ns_parts ? ns_parts + 1 : nullptr);
    if (st != XCCL_OK && flagged) {
        *flagged = 0;
    }
    return st;
}

void xccl_rocm_graph_cache_destroy(void)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return;
    }
    GraphCache                 &gc = g_graphs[dev];
    std::lock_guard<std::mutex> guard(gc.lock);
    for (GraphSlot &s : gc.slot) {
        if (s.live && s.last_stream_valid) {
            (void)hipStreamSynchronize(s.last_stream);
        }
        destroy_slot(s);
    }
}

void xccl_rocm_set_launch_shape(int blocks_per_cu, int resident_per_cu)
{
    read_env_once();
    g_resident.store(resident_per_cu > 0 ? resident_per_cu : 0, std::memory_order_release);
    g_blocks_per_cu.store(blocks_per_cu > 0 ? blocks_per_cu : kDefaultBlocksPerCu, std::memory_order_release);
    g_shape_epoch.fetch_add(1, std::memory_order_release); // plans cached by the threads are stale now
}

void xccl_rocm_set_slot_max_grid(int max_grid)
{
    read_env_once();
    g_slot_max_grid.store(max_grid >= 0 ? (unsigned)max_grid : kDefaultSlotMaxGrid, std::memory_order_release);
    g_shape_epoch.fetch_add(1, std::memory_order_release);
}

void xccl_rocm_set_burst_max_grid(int max_grid)
{
    read_env_once();
    g_burst_max_grid.store(max_grid >= 0 ? (unsigned)max_grid : 2048u, std::memory_order_release);
    g_shape_epoch.fetch_add(1, std::memory_order_release);
}

xccl_status_t xccl_rocm_reduce_multi_plan(void *sbuf1, void *sbuf2, void *rbuf, size_t count, size_t size,
                                          size_t stride, xccl_dt_t dtype, xccl_op_t op, unsigned *grid,
                                          unsigned *block, char *name, size_t name_len)
{
    Plan          plan;
    xccl_status_t st = make_plan(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, &plan);
    if (st != XCCL_OK) {
        return st;
    }
    if (grid) {
        *grid = plan.grid;
    }
    if (block) {
        *block = kBlock;
    }
    if (name && name_len > 0) {
        const char *n = hipKernelNameRefByPtr(plan.fn, nullptr);
        snprintf(name, name_len, "%s", n ? n : "");
    }
    return XCCL_OK;
}

xccl_status_t xccl_rocm_reduce_multi_route(void *sbuf1, void *sbuf2, void *rbuf, size_t count, size_t size,
                                           size_t stride, xccl_dt_t dtype, xccl_op_t op, int own_queue,
                                           unsigned *grid, unsigned *lds_bytes, int *burst, int *route)
{
    Plan          plan;
    xccl_status_t st = make_plan(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, &plan);
    if (st != XCCL_OK) {
        return st;
    }
    (void)direct_enabled(); // the own queues' environment
    const KernelEntry *e = lookup(dtype, op);
    if (grid) {
        *grid = plan.grid;
    }
    if (lds_bytes) {
        *lds_bytes = plan.lds_bytes;
    }
    if (burst) {
        *burst = plan.fn == e->fn_burst;
    }
    if (route) {
        *route = completion_route(plan, XCCL_ROCM_FLAG_WORDS, own_queue != 0, true, true);
    }
    return XCCL_OK;
}

xccl_status_t xccl_rocm_stream_gate(int *dev_flag, uint64_t max_ns, void *hip_stream)
{
    if (dev_flag == nullptr) {
        return XCCL_ERR_INVALID_PARAM;
    }
    // wall_clock64() counts at 100 MHz on gfx950.
    const uint64_t ticks = max_ns / 10 + 1;
    hipLaunchKernelGGL(stream_gate_kernel, dim3(1), dim3(1), 0, (hipStream_t)hip_stream, dev_flag, ticks);
    HIP_OR_FAIL(hipGetLastError());
    return XCCL_OK;
}

} // extern "C"
