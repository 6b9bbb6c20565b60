// graph_launch.hip -- the reduction launched as a cached single-kernel-node
// hipGraph (xccl_rocm_reduce_multi_graph* of include/xccl_rocm_kernels.h).
#include "launch_plan.hpp"

#include <mutex>
#include <string.h>

using namespace xccl_rocm;

namespace {

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

} // namespace

extern "C" {

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
} // extern "C"
