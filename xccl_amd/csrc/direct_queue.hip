// direct_queue.hip -- the component's own dispatch queues
// (xccl_rocm_reduce_multi_direct and its knobs, include/xccl_rocm_kernels.h).
#include "launch_plan.hpp"

#include <hsa/hsa.h>
#include <hsa/hsa_ext_amd.h>

#include <atomic>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>
#include <stdlib.h>
#include <string.h>
#if defined(__x86_64__) || defined(__i386__)
#include <immintrin.h>
#endif

using namespace xccl_rocm;

namespace {

// A reduction that reports its own completion -- a blocking call, or a
// stream-ordered one whose event is the completion word -- needs nothing of a
// HIP stream: no event, no ordering against other work.  Such launches go out
// as AQL packets on user-mode queues that the component creates through the
// HSA runtime (the layer HIP itself sits on): the host's part of a launch
// shrinks from ~2.6 us inside hipLaunchKernel, with its locks and pools, to
// writing 64 bytes and ringing a doorbell.  The kernels are the same code,
// loaded a second time from the bare code objects embedded in this library
// (kernel_images.S); they read no implicit launch arguments, so the kernel
// argument block is ReduceArgs and nothing else.  Packets carry agent-scope
// acquire and release fences, which is what a kernel launched on a HIP stream
// behind other kernels gets (system-scope acquire on request); the result
// stores are write-through and waited for by the kernel itself.  A
// stream-ordered launch carries the barrier bit, so that one thread's launches
// run in order; a blocking caller has waited for its own earlier launches and
// brings an argument block of its own, so its packet does not wait for other
// threads' launches on the same queue.
//   Two queues per device by default, shared by the component's four thread
// slots (slot s uses queue s mod 2), each created when a thread that uses it
// first calls, behind that slot's HIP stream.  Measured with the argument
// blocks in pinned host memory (in device memory, flush write included, every
// figure is about 0.5 us lower, and four threads see 6.0 / 6.6-8.0), blocking call, 4
// sources x 1 KiB, p50 / p99 in us, 1 / 2 / 4 calling threads: this 5.5 / 5.8,
// 6.3 / 8.7, 6.7-7.2 / 13.2; with the barrier bit on every packet 6.3 / 7.1,
// 6.1-6.4 / 8.8, 6.9-7.7 / 13.6; slots 2 and 3 on HIP streams instead 5.4 / 5.8,
// 7.1-7.3 / 10.9, 10.1-10.6 / 30-32; a queue per slot 5.4-5.8 / 6.1, 6.1-6.4 /
// 9.0, 7.7 / 21; one queue for all 5.8-6.3 / 7.2, 6.6 / 8.9, 12.4-12.9 / 13.4
// (the packet processor takes ~3 us per packet of a queue, fences included).
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
    // One producer at a time, from reserving a packet to ringing the doorbell for it.  The hardware queue would
    // take packets from several producers at once, but a tool that interposes on queue submission (a profiler's
    // intercept queue) then meets several new packets behind one doorbell, possibly across the ring's wrap; with
    // one producer at a time every doorbell stands for exactly one new packet, in index order.  The section is a
    // 64-byte store, the flush write for an argument block in device memory, and a doorbell write.
    std::atomic_flag turn = ATOMIC_FLAG_INIT;
};

struct QueueTurn {
    explicit QueueTurn(DirectQueue &dq) : dq_(dq)
    {
        while (dq_.turn.test_and_set(std::memory_order_acquire)) {
#if defined(__x86_64__) || defined(__i386__)
            _mm_pause();
#endif
        }
    }
    ~QueueTurn() { dq_.turn.clear(std::memory_order_release); }
    QueueTurn(const QueueTurn &)            = delete;
    QueueTurn &operator=(const QueueTurn &) = delete;
    DirectQueue &dq_;
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
    DirectKernel                                  tail_kernel{}; // xccl_rocm_tail_flag_kernel, looked up on first use
    // Kernel-argument blocks in DEVICE memory that the host writes through the PCIe aperture: a launch whose
    // arguments sit there starts 0.8 us sooner than one whose waves fetch them from pinned host memory (an
    // empty kernel's completion word is seen 3.7 us after the doorbell instead of 4.55).  Allocated once per
    // device and kept until the process ends, whatever happens to the queues.
    void                                         *arena       = nullptr;
    volatile uint32_t                            *hdp_flush   = nullptr; // the device's host-data-path flush register
    size_t                                        arena_bytes = 0;
    bool                                          arena_tried = false;
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
//   g_direct_tail     1: such launches stay on the own queue with a one-lane kernel as a second packet behind
//                     them that stores the completion word (XCCL_MC_ROCM_DIRECT_TAIL)
std::atomic<int>      g_direct_tail{1};
//   g_direct_confirm  what the host does between writing an argument block in device memory and ringing the
//                     doorbell, see before_doorbell (XCCL_MC_ROCM_DIRECT_CONFIRM, 0..3)
std::atomic<int>      g_direct_confirm{1};

// Host stores into device memory pass through the GPU's host data path, which may hold them back; the runtime
// names a register that, written, makes it pass them on (HSA_AMD_AGENT_INFO_HDP_FLUSH; the kernel driver and the
// HIP runtime write it after their own stores into device memory).  After an argument block in device memory has
// been written, before the doorbell:
//   mode 1  the stores leave the core (sfence), then that register is written: a posted write that reaches the
//           device behind the argument stores and ahead of the doorbell (default; +0.33 us per launch, measured)
//   mode 2  the same, and the register is read back, which returns when the flush has been carried out (+1.4 us)
//   mode 3  the block's last word is read back instead, which returns when the stores are in device memory
//           (+1.3-1.7 us)
//   mode 0  only the sfence (what the figures before this register was used were measured with: no stale
//           argument in some 10^7 launches, but nothing says the host data path may not hold a store back)
// Modes 2 and 3 cost more than keeping the blocks in pinned host memory (XCCL_MC_ROCM_DEVICE_KERNARG=0, +0.55 us).
inline void store_fence()
{
#if defined(__x86_64__) || defined(__i386__)
    _mm_sfence();
#else
    __atomic_thread_fence(__ATOMIC_SEQ_CST);
#endif
}

// The last step before the doorbell of a launch whose argument block (`block`, `bytes`) lies in device memory and
// has been written and fenced.  It comes behind the packet's own stores, so that it also covers a packet ring that
// the runtime keeps in device memory (HSA_ALLOCATE_QUEUE_DEV_MEM=1).
inline void before_doorbell(volatile uint32_t *hdp_flush, const void *block, size_t bytes)
{
    int mode = g_direct_confirm.load(std::memory_order_relaxed);
    if (mode == 0) {
        return;
    }
    if (hdp_flush == nullptr) {
        mode = 3; // no such register on this device: the read-back is what is left
    }
    store_fence(); // the packet's stores too, should they be write-combined stores into device memory
    if (mode == 1 || mode == 2) {
        *hdp_flush = 1u;
        if (mode == 2) {
            (void)*hdp_flush;
        }
    } else {
#if defined(__x86_64__) || defined(__i386__)
        _mm_mfence();
#endif
        (void)*reinterpret_cast<const volatile uint32_t *>(static_cast<const char *>(block) + bytes - 4);
    }
#if defined(__x86_64__) || defined(__i386__)
    if (mode == 1) {
        _mm_sfence();
    } else {
        _mm_mfence();
    }
#else
    __atomic_thread_fence(__ATOMIC_SEQ_CST);
#endif
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
        const char *t = getenv("XCCL_MC_ROCM_DIRECT_TAIL");
        if (t != nullptr) {
            g_direct_tail.store(atoi(t) != 0, std::memory_order_release);
        }
        const char *c = getenv("XCCL_MC_ROCM_DIRECT_CONFIRM");
        if (c != nullptr) {
            g_direct_confirm.store(atoi(c) < 0 || atoi(c) > 3 ? 1 : atoi(c), std::memory_order_release);
        }
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

#define HSA_OR_GIVE_UP_STATUS(call)            \
    do {                                       \
        if ((call) != HSA_STATUS_SUCCESS) {    \
            return XCCL_ERR_NO_RESOURCE;       \
        }                                      \
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

struct PoolSearch {
    hsa_agent_t           cpu;
    hsa_amd_memory_pool_t pool;
    bool                  ok;
};

hsa_status_t first_cpu(hsa_agent_t agent, void *data)
{
    hsa_device_type_t type;
    if (hsa_agent_get_info(agent, HSA_AGENT_INFO_DEVICE, &type) == HSA_STATUS_SUCCESS && type == HSA_DEVICE_TYPE_CPU) {
        static_cast<PoolSearch *>(data)->cpu = agent;
        return HSA_STATUS_INFO_BREAK;
    }
    return HSA_STATUS_SUCCESS;
}

// The device's ordinary (coarse-grained) memory pool, if the host may be given access to allocations from it.
hsa_status_t host_visible_device_pool(hsa_amd_memory_pool_t pool, void *data)
{
    PoolSearch       *want = static_cast<PoolSearch *>(data);
    hsa_amd_segment_t seg;
    uint32_t          flags = 0;
    bool              alloc = false;
    if (hsa_amd_memory_pool_get_info(pool, HSA_AMD_MEMORY_POOL_INFO_SEGMENT, &seg) != HSA_STATUS_SUCCESS ||
        seg != HSA_AMD_SEGMENT_GLOBAL ||
        hsa_amd_memory_pool_get_info(pool, HSA_AMD_MEMORY_POOL_INFO_GLOBAL_FLAGS, &flags) != HSA_STATUS_SUCCESS ||
        (flags & HSA_AMD_MEMORY_POOL_GLOBAL_FLAG_COARSE_GRAINED) == 0 ||
        hsa_amd_memory_pool_get_info(pool, HSA_AMD_MEMORY_POOL_INFO_RUNTIME_ALLOC_ALLOWED, &alloc) != HSA_STATUS_SUCCESS ||
        !alloc) {
        return HSA_STATUS_SUCCESS;
    }
    hsa_amd_memory_pool_access_t access = HSA_AMD_MEMORY_POOL_ACCESS_NEVER_ALLOWED;
    if (hsa_amd_agent_memory_pool_get_info(want->cpu, pool, HSA_AMD_AGENT_MEMORY_POOL_INFO_ACCESS, &access) != HSA_STATUS_SUCCESS ||
        access == HSA_AMD_MEMORY_POOL_ACCESS_NEVER_ALLOWED) {
        return HSA_STATUS_SUCCESS; // no large PCIe aperture on this system
    }
    want->pool = pool;
    want->ok   = true;
    return HSA_STATUS_INFO_BREAK;
}

// `bytes` of device memory the host can write, or NULL.  Caller holds dd.lock.
void *direct_arena(DirectDevice &dd, size_t bytes)
{
    if (dd.arena != nullptr) {
        return bytes <= dd.arena_bytes ? dd.arena : nullptr;
    }
    if (dd.arena_tried) {
        return nullptr;
    }
    dd.arena_tried = true;
    const char *off = getenv("XCCL_MC_ROCM_DEVICE_KERNARG");
    if (off != nullptr && atoi(off) == 0) {
        return nullptr;
    }
    PoolSearch want{};
    hsa_status_t it = hsa_iterate_agents(first_cpu, &want);
    if (it != HSA_STATUS_INFO_BREAK) {
        return nullptr;
    }
    it = hsa_amd_agent_iterate_memory_pools(dd.agent, host_visible_device_pool, &want);
    if ((it != HSA_STATUS_SUCCESS && it != HSA_STATUS_INFO_BREAK) || !want.ok) {
        return nullptr;
    }
    void *p = nullptr;
    if (hsa_amd_memory_pool_allocate(want.pool, bytes, 0, &p) != HSA_STATUS_SUCCESS || p == nullptr) {
        return nullptr;
    }
    hsa_agent_t both[2] = {want.cpu, dd.agent};
    if (hsa_amd_agents_allow_access(2, both, nullptr, p) != HSA_STATUS_SUCCESS) {
        (void)hsa_amd_memory_pool_free(p);
        return nullptr;
    }
    // the host's stores reach it and read back: otherwise pinned host memory stays the place
    volatile uint32_t *w = static_cast<volatile uint32_t *>(p);
    for (size_t i = 0; i < bytes / sizeof(uint32_t); ++i) {
        w[i] = 0;
    }
    w[0] = 0x5eed5eedu;
    __atomic_thread_fence(__ATOMIC_SEQ_CST);
    if (w[0] != 0x5eed5eedu) {
        (void)hsa_amd_memory_pool_free(p);
        return nullptr;
    }
    w[0] = 0;
    hsa_amd_hdp_flush_t hdp{};
    if (hsa_agent_get_info(dd.agent, (hsa_agent_info_t)HSA_AMD_AGENT_INFO_HDP_FLUSH, &hdp) == HSA_STATUS_SUCCESS) {
        dd.hdp_flush = hdp.HDP_MEM_FLUSH_CNTL;
    }
    dd.arena       = p;
    dd.arena_bytes = bytes;
    return p;
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

// Whether `p` lies in the device's arena of host-written device memory.
inline bool in_arena(const DirectDevice &dd, const void *p)
{
    const char *c = static_cast<const char *>(p);
    const char *a = static_cast<const char *>(dd.arena);
    return a != nullptr && c >= a && c < a + dd.arena_bytes;
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

    if (kernarg != nullptr) {
        // the caller's own argument block (its until the launch is complete).  It may be device memory behind a
        // write-combining mapping: its stores leave the core before the doorbell's does (posted writes to one
        // device arrive in order)
        memcpy(kernarg, &plan.args, sizeof(ReduceArgs));
        store_fence();
    }

    QueueTurn      turn(*dq);
    hsa_queue_t   *q   = dq->q;
    const uint64_t idx = hsa_queue_add_write_index_scacq_screl(q, 1);
    while (idx - hsa_queue_load_read_index_scacquire(q) >= q->size) {
        // queue full: kDirectPackets launches waiting to start; wait for the oldest
        if (g_direct_failed.load(std::memory_order_acquire) != 0) {
            return XCCL_ERR_NO_RESOURCE; // the queue is dead; the reserved packet stays invalid
        }
    }
    char *args = static_cast<char *>(kernarg);
    if (args == nullptr) {
        args = dq->kernarg + (idx & (kKernargSlots - 1)) * kKernargSlot; // the queue's own ring of argument blocks
        memcpy(args, &plan.args, sizeof(ReduceArgs));
    }

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
    if (in_arena(dd, kernarg)) {
        before_doorbell(dd.hdp_flush, kernarg, sizeof(ReduceArgs));
    }
    hsa_signal_store_screlease(q->doorbell_signal, (hsa_signal_value_t)idx);
    g_direct_launches.fetch_add(1, std::memory_order_relaxed);
    return XCCL_OK;
}

// The one-lane kernel that stores `seq` to `flag`, as a packet with the barrier
// bit on queue `slot`; `kernarg`: 16 bytes the caller keeps until it has run.
xccl_status_t direct_launch_tail(DirectDevice &dd, int slot, uint32_t *flag, uint32_t seq, void *kernarg)
{
    DirectQueue *dq = nullptr;
    if (slot < 0 || slot >= kMaxDirectQueues || kernarg == nullptr || !direct_queue(dd, slot, &dq)) {
        return XCCL_ERR_NO_RESOURCE;
    }
    if (__atomic_load_n(&dd.tail_kernel.object, __ATOMIC_ACQUIRE) == 0) {
        std::lock_guard<std::mutex> guard(dd.lock);
        if (dd.tail_kernel.object == 0) {
            hsa_executable_symbol_t sym;
            uint32_t                kernarg_bytes = 0, priv = 0;
            DirectKernel            k;
            HSA_OR_GIVE_UP_STATUS(hsa_executable_get_symbol_by_name(dd.exe, "xccl_rocm_tail_flag_kernel.kd", &dd.agent, &sym));
            HSA_OR_GIVE_UP_STATUS(hsa_executable_symbol_get_info(sym, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_OBJECT, &k.object));
            HSA_OR_GIVE_UP_STATUS(hsa_executable_symbol_get_info(sym, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_KERNARG_SEGMENT_SIZE, &kernarg_bytes));
            HSA_OR_GIVE_UP_STATUS(hsa_executable_symbol_get_info(sym, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_GROUP_SEGMENT_SIZE, &k.group));
            HSA_OR_GIVE_UP_STATUS(hsa_executable_symbol_get_info(sym, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_PRIVATE_SEGMENT_SIZE, &priv));
            if (kernarg_bytes > 16 || priv != 0 || k.object == 0) {
                return XCCL_ERR_NO_RESOURCE;
            }
            dd.tail_kernel.group = k.group;
            __atomic_store_n(&dd.tail_kernel.object, k.object, __ATOMIC_RELEASE);
        }
    }
    struct {
        uint32_t *flag;
        uint32_t  seq, pad;
    } args = {flag, seq, 0};
    memcpy(kernarg, &args, sizeof(args));
    store_fence();
    QueueTurn      turn(*dq);
    hsa_queue_t   *q   = dq->q;
    const uint64_t idx = hsa_queue_add_write_index_scacq_screl(q, 1);
    while (idx - hsa_queue_load_read_index_scacquire(q) >= q->size) {
        if (g_direct_failed.load(std::memory_order_acquire) != 0) {
            return XCCL_ERR_NO_RESOURCE;
        }
    }
    hsa_kernel_dispatch_packet_t *p = static_cast<hsa_kernel_dispatch_packet_t *>(q->base_address) + (idx & (q->size - 1));
    p->workgroup_size_x     = 1;
    p->workgroup_size_y     = 1;
    p->workgroup_size_z     = 1;
    p->reserved0            = 0;
    p->grid_size_x          = 1;
    p->grid_size_y          = 1;
    p->grid_size_z          = 1;
    p->private_segment_size = 0;
    p->group_segment_size   = dd.tail_kernel.group;
    p->kernel_object        = dd.tail_kernel.object;
    p->kernarg_address      = kernarg;
    p->reserved2            = 0;
    p->completion_signal.handle = 0;
    const uint32_t header = (uint32_t)HSA_PACKET_TYPE_KERNEL_DISPATCH << HSA_PACKET_HEADER_TYPE |
                            1u << HSA_PACKET_HEADER_BARRIER |
                            (uint32_t)HSA_FENCE_SCOPE_AGENT << HSA_PACKET_HEADER_SCACQUIRE_FENCE_SCOPE |
                            (uint32_t)HSA_FENCE_SCOPE_AGENT << HSA_PACKET_HEADER_SCRELEASE_FENCE_SCOPE;
    const uint32_t setup  = 1u << HSA_KERNEL_DISPATCH_PACKET_SETUP_DIMENSIONS;
    __atomic_store_n(reinterpret_cast<uint32_t *>(p), header | setup << 16, __ATOMIC_RELEASE);
    if (in_arena(dd, kernarg)) {
        before_doorbell(dd.hdp_flush, kernarg, sizeof(args));
    }
    hsa_signal_store_screlease(q->doorbell_signal, (hsa_signal_value_t)idx);
    return XCCL_OK;
}

// Waits until everything queued on `dq` has completed: a barrier packet with a
// completion signal goes in behind it (a stream-ordered launch whose event
// nobody waited for may still be queued or running when the component closes).
// Bounded: gives up after `limit_ns`, or when the queue has reported an error.
void direct_drain(DirectQueue &dq, uint64_t limit_ns)
{
    hsa_queue_t *q = dq.q;
    hsa_signal_t done{};
    if (g_direct_failed.load(std::memory_order_acquire) != 0 ||
        hsa_amd_signal_create(1, 0, nullptr, HSA_AMD_SIGNAL_AMD_GPU_ONLY, &done) != HSA_STATUS_SUCCESS) {
        return;
    }
    const uint64_t t0   = clock_ns();
    bool           room = true;
    {
        QueueTurn      turn(dq);
        const uint64_t idx = hsa_queue_add_write_index_scacq_screl(q, 1);
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
        }
    }
    while (room && hsa_signal_load_scacquire(done) != 0) {
        if (g_direct_failed.load(std::memory_order_acquire) != 0 || clock_ns() - t0 > limit_ns) {
            fprintf(stderr, "xccl mc_rocm: the component's dispatch queue did not drain; destroying it anyway\n");
            break;
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
            direct_drain(dq, 10000000000ull);
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
    dd.tail_kernel = DirectKernel{};
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

namespace xccl_rocm {

void direct_read_env()
{
    (void)direct_enabled();
}

bool direct_signal_enabled()
{
    return g_direct_signal.load(std::memory_order_relaxed) != 0;
}

bool direct_tail_enabled()
{
    return g_direct_tail.load(std::memory_order_relaxed) != 0;
}

// Loading the code and creating a queue takes milliseconds, which belong into a
// device's set-up and not into the first small reduction; failure leaves the
// stream path.  Only queue 0: the others are created when a thread that uses
// them first calls.  (The device serves the queue created last fastest: an
// empty kernel's completion word is seen 4.6 us after the doorbell on the
// newest of up to 12 open queues, 4.8-5.5 us on the older ones.)
void direct_prepare_first_queue()
{
    DirectDevice *dd = direct_device();
    DirectQueue  *dq = nullptr;
    if (dd != nullptr && !direct_queue(*dd, 0, &dq)) {
        dd->state.store(-1, std::memory_order_release);
    }
}

} // namespace xccl_rocm

extern "C" {

void *xccl_rocm_direct_kernarg_arena(size_t bytes)
{
    DirectDevice *dd = direct_device();
    if (dd == nullptr || bytes == 0) {
        return nullptr;
    }
    std::lock_guard<std::mutex> guard(dd->lock);
    return direct_arena(*dd, bytes);
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
    if (route == XCCL_ROCM_ROUTE_TAIL) {
        // the reduction, then a one-lane kernel behind it that stores the word; its 16 bytes of arguments sit
        // behind the reduction's in the caller's block
        if (kernarg == nullptr) {
            return XCCL_OK;
        }
        static_assert(sizeof(ReduceArgs) + 16 <= XCCL_ROCM_KERNARG_BYTES, "room for the tail kernel's arguments");
        if (direct_launch(*dd, queue_slot, plan, 0, ordered, kernarg) != XCCL_OK) {
            return XCCL_OK;
        }
        if (direct_launch_tail(*dd, queue_slot, dev_flag, seq, static_cast<char *>(kernarg) + XCCL_ROCM_KERNARG_BYTES - 16) !=
            XCCL_OK) {
            // the reduction is queued but no kernel will tell when it is over: wait for the queue to drain and
            // store the word from here (it is host memory, at the same address on both sides)
            DirectQueue *dq = nullptr;
            if (direct_queue(*dd, queue_slot, &dq)) {
                direct_drain(*dq, 10000000000ull);
            }
            __atomic_store_n(dev_flag, seq, __ATOMIC_RELEASE);
        }
        *flagged = 1;
        return XCCL_OK;
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
void xccl_rocm_set_direct_confirm(int on)
{
    (void)direct_enabled();
    g_direct_confirm.store(on < 0 || on > 3 ? 1 : on, std::memory_order_release);
}

void xccl_rocm_set_direct_tail(int on)
{
    (void)direct_enabled();
    g_direct_tail.store(on != 0, std::memory_order_release);
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
    (void)direct_enabled(); // the environment first, so that it does not overwrite this later
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
} // extern "C"
