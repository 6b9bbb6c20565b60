// launch_plan.hpp -- what the host-side translation units of the kernel ABI
// (include/xccl_rocm_kernels.h) share: reduce_launch.hip plans a call and
// launches it on a HIP stream, graph_launch.hip launches the same plan as a
// cached one-node hipGraph, direct_queue.hip puts it on the component's own
// AQL queues.
#ifndef XCCL_ROCM_LAUNCH_PLAN_HPP_
#define XCCL_ROCM_LAUNCH_PLAN_HPP_

#include "reduce_kernel.hpp"
#include "xccl_rocm_kernels.h"

#include <stdint.h>
#include <stdio.h>

namespace xccl_rocm {

constexpr int    kMaxDevices  = 64;
constexpr size_t kLdsPerGroup = 64 * 1024; // most LDS a workgroup may ask for

// Launches of at most this many workgroups may count their own arrivals for a
// completion word when nothing else can write it: each workgroup pays an
// atomic on one of 64 shared counters (~12 ns per arrival on the same word,
// measured), which beats the queue's completion signal up to here and would
// serialise a grid of hundreds of thousands.
constexpr unsigned kMaxFlaggedGrid = 8192;

// One launch: kernel, grid of one-wave workgroups, and its argument block.
struct Plan {
    const void *fn;
    unsigned    grid;
    unsigned    lds_bytes; // dynamic LDS asked for only to bound resident workgroups per CU
    ReduceArgs  args;
};

// Plan of a call (the calling thread's last plan is reused when the arguments
// repeat), or `*nothing` when there is nothing to launch: size == 0 is a no-op
// for a supported pair, reference mem_component.c:129-131.
xccl_status_t prepare(void *s1, void *s2, void *dst, size_t count, size_t size, size_t stride, xccl_dt_t dt,
                      xccl_op_t op, Plan *plan, bool *nothing);

// How the host learns that the launch of `plan` is complete (XCCL_ROCM_ROUTE_*),
// and the arming of a plan whose kernel writes its own completion word (routes
// SLOTS and COUNTED; returns the number of words the host has to watch).
int completion_route(const Plan &plan, uint32_t flag_words, bool own_queue, bool want_flag, bool has_signal);
int arm_completion(Plan &plan, int route, uint32_t *dev_count, uint32_t *dev_flag, uint32_t seq);

uint64_t clock_ns(); // CLOCK_MONOTONIC

// direct_queue.hip
void direct_read_env();            // reads the own queues' environment variables, once
bool direct_signal_enabled();      // large launches may complete through a packet's completion signal
bool direct_tail_enabled();        // ... or through a one-lane kernel as a second packet behind them
void direct_prepare_first_queue(); // loads the kernels' code objects and creates queue 0 of the current device

#define HIP_OR_FAIL(call)                                                                          \
    do {                                                                                           \
        hipError_t e_ = (call);                                                                    \
        if (e_ != hipSuccess) {                                                                    \
            fprintf(stderr, "xccl mc_rocm: %s failed: %s\n", #call, hipGetErrorString(e_));        \
            return XCCL_ERR_NO_MESSAGE;                                                            \
        }                                                                                          \
    } while (0)

} // namespace xccl_rocm
#endif // XCCL_ROCM_LAUNCH_PLAN_HPP_
