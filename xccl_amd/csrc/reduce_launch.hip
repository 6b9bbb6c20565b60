// reduce_launch.hip -- host side of the kernel ABI declared in
// include/xccl_rocm_kernels.h: (dtype, op) -> kernel lookup, launch planning,
// completion routes, the launch on a HIP stream, the entry that allocates
// nothing, and the stream gate.  The cached one-node hipGraph launch is in
// graph_launch.hip, the component's own dispatch queues in direct_queue.hip.
#include "launch_plan.hpp"

#include <atomic>
#include <mutex>
#include <stdlib.h>
#include <string.h>
#include <time.h>

namespace xccl_rocm {
namespace {

// Grid cap in workgroups per compute unit.  Large on purpose: one tile per
// workgroup measured fastest, so the cap only bounds the grid of huge calls.
constexpr int kDefaultBlocksPerCu = 8192;

// Resident one-wave workgroups per compute unit for large launches (0 = the
// defaults of lds_for_resident, > 0 = this many for every call,
// >= kNoResidentCap = no cap).
constexpr int    kNoResidentCap = 32;
constexpr size_t kLdsPerCu      = 160 * 1024;

// Hard bound of what XCCL_MC_ROCM_MAX_COUNTED_GRID may ask for (measurement; the two-level count itself has no limit).
constexpr unsigned kMaxCountedGridKnob = 1u << 20;

std::atomic<int> g_blocks_per_cu{-1}; // -1: not read from the environment yet
std::atomic<int> g_resident{0};
std::atomic<int> g_tail_flag{1};
std::atomic<unsigned> g_shape_epoch{0}; // bumped when a launch-shape knob changes
// The same bound for launches on the component's own dispatch queue, where a larger launch gets a one-lane kernel
// as a second packet behind it.  With the kernel arguments in device memory that second packet costs less than the
// second level of arrival counting (grids beyond 64 workgroups count in two levels): blocking call, us, counting /
// second packet, 2 | 8 sources: 32 workgroups 5.49 / 5.77 | 5.64 / 5.91, 64: 5.51 / 5.83 | 5.83 / 5.91, 96: 5.83 /
// 5.83 | 5.99 / 5.87, 256: 5.83 / 5.83 | 6.02 / 5.92, 1024: 6.22 / 5.87 | 6.61 / 6.37, 2048: 6.58 / 6.33 | 7.43 /
// 6.73, 4096: 7.34 / 6.76 | 9.45 / 9.25, 8192: 8.83 / 7.76 | 16.0 / 15.2.  (With that option off the bound that
// serves is 6144: counting against the HIP stream's queued kernel.)
constexpr unsigned kCountedGridUnset = ~0u; // 64 with the second packet, 6144 without
std::atomic<unsigned> g_direct_counted_grid{kCountedGridUnset};
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


// LDS per workgroup that lets `resident` workgroups share a compute unit.
// `footprint`: bytes the call touches.  Measured (fp32 SUM, destination
// rotating through 4 vectors so that the 256 MB memory-side cache cannot keep
// it; GB/s at 12 / 13 / 14 / 15 / 16 / 17 / 18 / 20 / 22 resident and without
// a bound):
//    2 sources x 256 MiB: every wave slot (7.0 TB/s against 6.4 at 16)
//    3 x 256 MiB   6205 6365 6570 6570 6655 6655 6620 6630 6530 | 6605   (same destination every launch:
//                  20 and more 7280-7450, 16: 6965 -- hence 20)
//    4 x 256 MiB   6210 6390 6560 6555 6680 6685 6565 6570 6510 | 6685
//    5 x 256 MiB   6675 6790 6665 6650 6530 6510 6490 6475 6435 | 6520
//    8 x 256 MiB   6545 6700 6770 6760 6685 6695 6585 6585 6485 | 6710   (same destination: 16-17 6875-6895,
//                  15: 6850, 14: 6825)
//    8 x 1 GiB     6545 6735 6700 6725 6630 6625 6560 6570 6505 | 6635
//   12 x 128 MiB   6610 6770 6775 6810 6690 6665 6610 6625 6510 | 6640
//   16 x 128 MiB   6515 6695 6760 6765 6650 6645 6555 6565 6470 | 6595
//    8 x 64 MiB    6475 6590 6675 6670 6820 6815 6800 6795 6800 | 6775
// A call whose vectors all fit the memory-side cache (the integer sweep's
// 16 Mi-element vectors of 1 and 2 bytes) is served from there when its
// operands were just written, and wants every slot as well (int8 SUM, 4
// sources: 6.86 TB/s against 6.26 at 16).
unsigned lds_for_resident(uint32_t nsrc, size_t grid, int cus, size_t footprint)
{
    int cap = g_resident.load(std::memory_order_relaxed);
    if (cap == 0) {
        // 8 and more sources want the bound from 8 MiB vectors on (16 sources x 8 MiB: 6.85 TB/s against
        // 6.36 without, 8 x 8 MiB: 6.62 against 6.46), fewer sources only once the call outgrows the cache
        const size_t fits = (size_t)(nsrc >= 8 ? 64 : 192) << 20;
        cap = (nsrc <= 2 || footprint <= fits) ? kNoResidentCap : nsrc == 3 ? 20 : nsrc == 4 ? 16 : nsrc < 8 ? 14 : 15;
        if (nsrc >= 8 && footprint <= ((size_t)1 << 30)) {
            cap = 16; // 8 x 64 MiB: 16 and more (table above); between 64 MiB and 1 GiB of footprint 16 is at least as good
        }
    }
    if (cap >= kNoResidentCap || grid <= (size_t)cap * (size_t)cus) {
        return 0; // the whole grid is resident at once anyway
    }
    size_t lds = (kLdsPerCu / (size_t)cap) & ~(size_t)511;
    return (unsigned)(lds > kLdsPerGroup ? kLdsPerGroup : lds); // 1 or 2 asked for: 2.5 is the fewest LDS can enforce
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

uint64_t clock_ns()
{
    timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (uint64_t)ts.tv_sec * 1000000000ull + (uint64_t)ts.tv_nsec;
}

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
// How the host learns that a launch is complete (values of XCCL_ROCM_ROUTE_*):
// one word per workgroup for a handful of workgroups, a word written by the
// last workgroup to arrive for small grids, and for larger ones a one-lane
// kernel queued behind the launch (on a HIP stream, or as a second packet on
// the component's own queue) or the packet's completion signal on the own
// queue; else the stream itself.
int completion_route(const Plan &plan, uint32_t flag_words, bool own_queue, bool want_flag, bool has_signal)
{
    if (!want_flag) {
        return XCCL_ROCM_ROUTE_STREAM;
    }
    const bool     tail_ok   = g_tail_flag.load(std::memory_order_relaxed) != 0;
    unsigned       own_bound = g_direct_counted_grid.load(std::memory_order_relaxed);
    if (own_bound == kCountedGridUnset) {
        own_bound = direct_tail_enabled() ? 64u : 6144u;
    }
    const unsigned counted   = own_queue ? own_bound
                               : tail_ok ? g_max_counted_grid.load(std::memory_order_relaxed)
                                         : kMaxFlaggedGrid;
    const unsigned slots_max = flag_words < XCCL_ROCM_FLAG_WORDS ? flag_words : XCCL_ROCM_FLAG_WORDS;
    if (plan.grid <= counted) {
        // a grid of one needs neither counting nor a second word: it stays on the counting path, which then has no atomics
        const bool by_slots = plan.grid > 1 && plan.grid <= slots_max && plan.grid <= g_slot_max_grid.load(std::memory_order_relaxed);
        return by_slots ? XCCL_ROCM_ROUTE_SLOTS : XCCL_ROCM_ROUTE_COUNTED;
    }
    if (own_queue) {
        if (direct_tail_enabled()) {
            return XCCL_ROCM_ROUTE_TAIL;
        }
        return has_signal && direct_signal_enabled() ? XCCL_ROCM_ROUTE_SIGNAL : XCCL_ROCM_ROUTE_STREAM;
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

} // namespace xccl_rocm

using namespace xccl_rocm;

namespace {

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
        direct_prepare_first_queue();
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
    direct_read_env();
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
