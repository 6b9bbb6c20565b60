/*
 * xccl_rocm_kernels.h -- the C ABI between the C host side of the ROCm
 * memory component and its gfx950 HIP kernels.
 *
 * It takes the place of the two `extern "C"` launchers the reference's CUDA
 * component declares for itself (src/utils/cuda/cuda_mem_component.c:110-125)
 * and defines in src/utils/cuda/kernels/xccl_cuda_reduce.cu:105-133 and
 * xccl_cuda_reduce_multi.cu:110-142.  Differences that a caller can see:
 *
 *   - every function here only ENQUEUES work on `hip_stream` (a hipStream_t
 *     passed as void*; NULL is the legacy default stream).  The reference
 *     launchers end with cudaStreamSynchronize; here waiting is the caller's
 *     business (the component's synchronous vtable entries do it).
 *   - `stride` is used in bytes exactly as given; it need not be a multiple
 *     of the element size (the reference asserts that it is).
 *   - fold order and operand order follow the reference's HOST path
 *     (src/utils/mem_component.c:133-139): acc = OP(sbuf1, sbuf2{0}), then
 *     acc = OP(sbuf2{j}, acc) for j = 1 .. count-1.  count == 0 behaves as
 *     count == 1, as it does there.
 *   - datatype coverage is INT8..INT64, UINT8..UINT64 (10 ops) and
 *     FLOAT16/32/64 (MAX, MIN, SUM, PROD); everything else returns
 *     XCCL_ERR_UNSUPPORTED (the reference kernels' convention).
 *
 * No pointer needs any alignment beyond what the caller already has.  rbuf /
 * target may be exactly sbuf1 or exactly sbuf2 (vector 0) -- the two in-place
 * forms the UCX team library uses (allreduce_knomial.c:118-121,
 * reduce_linear.c:28-34) -- and must not overlap a source in any other way
 * (the reference accumulates in rbuf, so with rbuf on a later vector of sbuf2
 * it reads its own partial result; that artefact is not reproduced).
 */
#ifndef XCCL_ROCM_KERNELS_H_
#define XCCL_ROCM_KERNELS_H_

#include "xccl_rocm_types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Looks up what the launchers need to know about the CURRENT device (its
 * compute-unit count, the address of the library's static counter array on
 * it) so that later calls on that device make no runtime query, and sets up
 * the dispatch queues of xccl_rocm_reduce_multi_direct there (loads the
 * kernels' code objects, creates the queues: milliseconds, and allocations).
 * Optional: the launchers do the same on their first call on a device; a
 * caller that will launch from inside a stream capture calls this once
 * outside it.  The component calls it when it sets a device up. */
xccl_status_t xccl_rocm_prepare_device(void);

/* XCCL_OK if a kernel exists for (dtype, op), XCCL_ERR_UNSUPPORTED if not.
 * Host-only; touches no device.  Same matrix as the two launchers below. */
xccl_status_t xccl_rocm_reduce_supported(xccl_dt_t dtype, xccl_op_t op);

/* target[i] = OP(sbuf1[i], sbuf2[i]), i < count.
 * Replaces xccl_cuda_reduce_impl (xccl_cuda_reduce.cu:105-133). */
xccl_status_t xccl_rocm_reduce_impl(void *sbuf1, void *sbuf2, void *target,
                                    size_t count, xccl_dt_t dtype,
                                    xccl_op_t op, void *hip_stream);

/* rbuf = sbuf1 OP sbuf2{0} OP ... OP sbuf2{count-1}; `size` elements per
 * vector, vectors of sbuf2 `stride` bytes apart.  One kernel launch, every
 * source read once, accumulator in registers.
 * Replaces xccl_cuda_reduce_multi_impl (xccl_cuda_reduce_multi.cu:110-142). */
xccl_status_t xccl_rocm_reduce_multi_impl(void *sbuf1, void *sbuf2, void *rbuf,
                                          size_t count, size_t size,
                                          size_t stride, xccl_dt_t dtype,
                                          xccl_op_t op, void *hip_stream);

/*
 * xccl_rocm_reduce_multi_impl with a completion word: `seq` is stored to
 * `*dev_flag` -- the device view of a host-mapped 32-bit word -- once the
 * last result store is visible system-wide, and `*flagged` is set to 1; the
 * caller may then poll the host view of the word instead of the stream (the
 * host sees the word 3-5 us before the queue's completion signal).  A small
 * launch writes the word itself: its workgroups count their arrivals in
 * `dev_count`, XCCL_ROCM_DONE_COUNT_BYTES of zeroed device memory (two
 * levels, one counter per 128-byte line), which the kernel leaves zero again.
 * Behind a larger launch (more than 2048 workgroups; XCCL_MC_ROCM_MAX_COUNTED_GRID)
 * a one-lane kernel is queued that stores the word: every result store of
 * the reduction is a system-scope write-through store, so the results are in
 * memory when that kernel starts.  With XCCL_MC_ROCM_TAIL_FLAG=0 in the
 * environment launches count their arrivals up to 8192 workgroups instead;
 * beyond that, or if the queued kernel's launch fails, `*flagged` is 0 and
 * the caller waits for the stream as usual.  One launch at a time per
 * (count, flag) pair.  No counterpart in the reference.
 */
#define XCCL_ROCM_DONE_COUNT_BYTES ((1 + 64) * 128)
xccl_status_t xccl_rocm_reduce_multi_flagged(void *sbuf1, void *sbuf2, void *rbuf,
                                             size_t count, size_t size,
                                             size_t stride, xccl_dt_t dtype,
                                             xccl_op_t op, void *hip_stream,
                                             uint32_t *dev_count,
                                             uint32_t *dev_flag, uint32_t seq,
                                             int *flagged);

/*
 * xccl_rocm_reduce_multi_flagged for a caller whose completion word is the
 * first of `flag_words` consecutive 32-bit words (host-mapped, device view in
 * `dev_flag`).  A launch of 2 to 8 workgroups (XCCL_MC_ROCM_SLOT_MAX_GRID, at
 * most min(flag_words, XCCL_ROCM_FLAG_WORDS)) then reports completion without
 * any counting: workgroup b stores `seq` to dev_flag[b] once its own result
 * stores are in memory, `*flagged` is set to the number of workgroups, and
 * the launch is complete when the first `*flagged` words all hold `seq`
 * (words beyond keep what earlier launches left there: compare for equality
 * with a `seq` that differs from launch to launch).  That spares such a launch
 * the round trip of an arrival atomic: blocking call, 2 sources x 2 KiB
 * 6.8-7.1 -> 6.4 us, 8 sources x 8 KiB 7.6-7.9 -> 7.4-7.5 us; every further
 * word costs the host's view about 0.1 us, so that from 12 workgroups on
 * counting is as fast and from 16 on faster (2 x 16 KiB: 7.7 against 7.9 us).
 * Every other launch behaves as under xccl_rocm_reduce_multi_flagged and sets
 * `*flagged` to 1 or 0.  No counterpart in the reference.
 */
#define XCCL_ROCM_FLAG_WORDS 16
xccl_status_t xccl_rocm_reduce_multi_slots(void *sbuf1, void *sbuf2, void *rbuf,
                                           size_t count, size_t size,
                                           size_t stride, xccl_dt_t dtype,
                                           xccl_op_t op, void *hip_stream,
                                           uint32_t *dev_count,
                                           uint32_t *dev_flag, uint32_t flag_words,
                                           uint32_t seq, int *flagged);

/*
 * xccl_rocm_reduce_multi_slots on the component's own dispatch queue instead
 * of a HIP stream, for callers that wait for the completion word and need no
 * stream order (the blocking entries of the vtable).  The launch goes out as
 * an AQL packet on one of up to four user-mode queues (`queue_slot` 0..3; by
 * default there are two, which slots 2 and 3 share with slots 0 and 1, see
 * xccl_rocm_set_direct_options) that
 * the component creates through the HSA runtime on first use; the host's part
 * of the launch is writing the packet and ringing the doorbell.  Launches of
 * one queue run in order, except that a `blocking` caller's launch -- the
 * caller waits for it before it issues anything else -- may be allowed not to
 * wait for other callers' launches on the same queue; they are not ordered
 * against any HIP stream: issue one only when everything it depends on is
 * complete, and wait for its completion before anything depends on it.
 * `kernarg`: XCCL_ROCM_KERNARG_BYTES of pinned host memory, or of
 * xccl_rocm_direct_kernarg_arena, that stay the caller's until the launch is
 * complete (NULL: a ring of the queue's own, and the launch is ordered).
 * `*flagged` > 0: launched, complete when the first `*flagged` words at
 * `dev_flag` hold `seq`: written by the launch itself up to 64 workgroups, by
 * a one-lane kernel that goes out as a second packet behind it beyond
 * (xccl_rocm_set_direct_tail; needs `kernarg`).  `*flagged` == -1: launched,
 * too large to count its own workgroups, the second packet switched off and
 * completion by signal switched on: complete when
 * xccl_rocm_direct_signal_done(*signal) -- `*signal` is created on first need
 * (0 before) and belongs to the queues: it goes with
 * xccl_rocm_direct_queue_destroy.  `*flagged` == 0 with XCCL_OK: nothing was
 * launched and the caller uses xccl_rocm_reduce_multi_slots instead -- the
 * call is too large for its own word (more than 6144 workgroups then) and
 * both of those are off, has size 0, the slot has no queue, the queue could
 * not be set up (said once on stderr), or the path is switched off
 * (XCCL_MC_ROCM_DIRECT_QUEUE=0 or xccl_rocm_set_direct_queue(0)).  Blocking
 * call, 4 sources x 1 KiB: p50 4.6 us against 7.1 us on a HIP stream, p99 4.8
 * against 10-12 us; 8 sources x 16 MiB: 26.4-26.9 against 28.4-28.8 us.  No
 * counterpart in the reference.
 */
#define XCCL_ROCM_KERNARG_BYTES 128
xccl_status_t xccl_rocm_reduce_multi_direct(void *sbuf1, void *sbuf2, void *rbuf,
                                            size_t count, size_t size,
                                            size_t stride, xccl_dt_t dtype,
                                            xccl_op_t op, int queue_slot,
                                            uint32_t *dev_count,
                                            uint32_t *dev_flag, uint32_t flag_words,
                                            uint32_t seq, uint64_t *signal,
                                            void *kernarg, int blocking,
                                            int *flagged);

/* `bytes` of DEVICE memory on the current device that the host can write
 * through the PCIe aperture, for the `kernarg` blocks of
 * xccl_rocm_reduce_multi_direct: a launch whose arguments sit there starts
 * 0.8 us sooner than one whose waves fetch them from pinned host memory (an
 * empty kernel's completion word is seen 3.7 us after the doorbell instead of
 * 4.55).  One arena per device, allocated on the first call and kept until
 * the process ends (later calls return the same memory if it is large enough);
 * NULL where the device's memory is not host-accessible, the own queues are
 * off or could not be set up, or XCCL_MC_ROCM_DEVICE_KERNARG=0: the caller
 * then brings pinned host memory. */
void *xccl_rocm_direct_kernarg_arena(size_t bytes);

/* Nonzero once the launch that armed `signal` (see above) is complete. */
int xccl_rocm_direct_signal_done(uint64_t signal);

/*
 * How the component's own queues are used; a negative (for `queues`: out of
 * range) argument leaves that setting alone.  Each also has an environment
 * variable, read once.
 *   acquire_system  1: launches carry a system-scope acquire fence instead of
 *                   an agent-scope one (XCCL_MC_ROCM_DIRECT_ACQUIRE=system)
 *   queues          1..4 queues per device, for thread slots 0..queues-1
 *                   (XCCL_MC_ROCM_DIRECT_QUEUES)
 *   share           1 (default): the other thread slots share those queues;
 *                   0: they keep to their HIP streams
 *                   (XCCL_MC_ROCM_DIRECT_SHARE)
 *   barrier         0 (default): a blocking caller's launch does not wait for
 *                   other callers' launches on its queue; 1: every launch
 *                   waits for all before it (XCCL_MC_ROCM_DIRECT_BARRIER)
 *   signal          1: launches too large to count their own workgroups stay
 *                   on these queues and complete through a completion signal;
 *                   0 (default): they go to the HIP stream
 *                   (XCCL_MC_ROCM_DIRECT_SIGNAL)
 * Measured with the kernel arguments still in pinned host memory (in device
 * memory, with the flush write of xccl_rocm_set_direct_confirm, every row is
 * 0.5 us lower and the shipped setting gives 4.8 / 5.0-6.1, 5.7 / 6.2-7.3,
 * 6.0 / 6.6-8.0), blocking call, 4 sources x 1 KiB,
 * p50 / p99 in us, 1 / 2 / 4
 * calling threads: two queues shared, no barrier 5.5 / 5.8, 6.3 / 8.7,
 * 6.7-7.2 / 13.2; shared, with barrier 6.3 / 7.1, 6.1-6.4 / 8.8, 6.9-7.7 /
 * 13.6; two queues not shared (threads 3 and 4 on HIP streams) 5.4 / 5.8,
 * 7.1-7.3 / 10.9, 10.1-10.6 / 30-32; four queues, no barrier 5.4-5.8 / 6.1,
 * 6.1-6.4 / 9.0, 7.7 / 21; one queue shared by all 5.8-6.3 / 7.2, 6.6 / 8.9,
 * 12.4-12.9 / 13.4.  A system-scope acquire costs 0.85 us on a 1 KiB call
 * and 2.5 us on 8 sources x 32 KiB.  Completion by signal is no faster than
 * the HIP stream with a queued one-lane kernel (8 sources x 16 MiB: 28.9-29.0
 * against 28.4-28.8 us per blocking call, kernel 22.4; x 64 MiB: 96.8-97.0
 * against 94.7-96.4, kernel 88.0).
 */
void xccl_rocm_set_direct_options(int acquire_system, int queues, int share,
                                  int barrier, int signal);

/* 1 (default): a launch too large to count its own workgroups stays on the
 * own queue, with a one-lane kernel as a second packet behind it that stores
 * the completion word (`*flagged` == 1 from xccl_rocm_reduce_multi_direct);
 * 0: it goes to the HIP stream (or completes by signal, above).  Also
 * XCCL_MC_ROCM_DIRECT_TAIL.  Blocking call, us, this / HIP stream with a
 * queued one-lane kernel / completion signal, 8 sources x 8 MiB 15.4 / 17.3 /
 * 16.6, x 16 MiB 26.4 / 28.8 / 27.7, x 64 MiB 93.5 / 95.8 / 94.6, x 256 MiB
 * 353.7 / 357.8 / 355.2; 2 sources x 8 MiB 7.7 / 9.7 / 8.8. */
void xccl_rocm_set_direct_tail(int on);

/* What the host does between writing an argument block that lies in device
 * memory and ringing the doorbell.  Host stores into device memory pass
 * through the GPU's host data path, which may hold them back until it is
 * flushed.  1 (default): write the device's flush register
 * (HSA_AMD_AGENT_INFO_HDP_FLUSH), a posted write that arrives behind the
 * argument stores and ahead of the doorbell; 2: also read that register back
 * (returns when the flush is done); 3: read the block's last word back
 * instead (returns when the stores are in device memory); 0: nothing but a
 * store fence.  Measured per small call: 0: 4.6 us, 1: 4.9, 2: 6.0, 3: 6.3,
 * blocks in pinned host memory (XCCL_MC_ROCM_DEVICE_KERNARG=0): 5.4.  Also
 * XCCL_MC_ROCM_DIRECT_CONFIRM. */
void xccl_rocm_set_direct_confirm(int mode);

/* Launches that went out on the component's own queues so far (all devices). */
uint64_t xccl_rocm_direct_launch_count(void);

/* Nonzero once one of those queues has reported an error (a launch on it may
 * then never complete): callers polling a completion word give up. */
int xccl_rocm_direct_queue_failed(void);

/* Switches the path on or off for the process (default on). */
void xccl_rocm_set_direct_queue(int on);

/* Destroys the current device's queues, their completion signals and the code
 * loaded for them, after waiting (bounded: 10 s, or until a queue reports an
 * error) for everything queued there to complete; the caller issues nothing
 * more while it runs.  Called by the component's close(). */
void xccl_rocm_direct_queue_destroy(void);

/*
 * xccl_rocm_reduce_multi_flagged for callers that must not allocate: code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  It has no counterpart in the reference.  The arrival counters
 * live in a static device array inside the library (XCCL_ROCM_DONE_COUNT_BYTES
 * per GPU, held until the process ends) instead of coming from the caller, and
 * the call allocates nothing: it enqueues one small kernel that clears the
 * counters and the reduction itself, which always counts its own workgroups
 * and stores `seq` to `*dev_flag` (caller-owned, device-visible) when the last
 * one is through.  Limit: at most 8192 workgroups, i.e. 8 MiB per vector; a
 * larger call returns XCCL_ERR_INVALID_PARAM and prints why.  Every call on a
 * GPU shares that GPU's array: calls that overlap in time on one GPU race.
 * The array's address on a device is looked up on the first call there (or by
 * xccl_rocm_prepare_device): make that one outside any capture.
 */
xccl_status_t xccl_rocm_reduce_multi_flagged_static(void *sbuf1, void *sbuf2, void *rbuf,
                                                    size_t count, size_t size,
                                                    size_t stride, xccl_dt_t dtype,
                                                    xccl_op_t op, void *hip_stream,
                                                    uint32_t *dev_flag, uint32_t seq);

/* Same contract and same kernel as xccl_rocm_reduce_multi_impl, but enqueued
 * as one launch of a pre-instantiated single-kernel-node hipGraph whose node
 * parameters are patched per call (a small per-device cache keeps the most
 * recent argument sets instantiated, so a k-nomial step that repeats with the
 * same buffers replays its graph untouched).  No counterpart in the
 * reference.  Calls on one device serialise on an internal lock. */
xccl_status_t xccl_rocm_reduce_multi_graph(void *sbuf1, void *sbuf2, void *rbuf,
                                           size_t count, size_t size,
                                           size_t stride, xccl_dt_t dtype,
                                           xccl_op_t op, void *hip_stream);

/* The graph launch with the completion word of xccl_rocm_reduce_multi_flagged
 * (launches of up to 8192 workgroups; `*flagged` tells) and, for measurement,
 * the host time of its steps in `ns_parts` (may be NULL; 4 values:
 * planning, lock + slot search, building or patching the graph -- which
 * first waits for the slot's previous launch --, hipGraphLaunch).  The sequence number is a kernel argument, so a flagged
 * launch patches its node on every call. */
xccl_status_t xccl_rocm_reduce_multi_graph_flagged(void *sbuf1, void *sbuf2, void *rbuf,
                                                   size_t count, size_t size,
                                                   size_t stride, xccl_dt_t dtype,
                                                   xccl_op_t op, void *hip_stream,
                                                   uint32_t *dev_count,
                                                   uint32_t *dev_flag, uint32_t seq,
                                                   int *flagged, uint64_t *ns_parts);

/* Drop every cached graph of the current device (component close). */
void xccl_rocm_graph_cache_destroy(void);

/*
 * Launch-shape knobs, for measurement.  `blocks_per_cu` caps the grid at
 * blocks_per_cu x (compute units) workgroups of one wavefront; beyond the cap
 * workgroups loop over tiles.  0 restores the built-in default (a cap large
 * enough that every tile gets its own workgroup).  `resident_per_cu`: how
 * many workgroups may be resident on a compute unit at once (enforced by
 * asking for LDS the kernel never touches); 0 = the built-in choice by source
 * count (16 to 32), 32 or more = no limit, 1 and 2 behave as 3 (a workgroup
 * cannot ask for more than 64 KiB).  Both are process-global and may also be
 * set through the environment (XCCL_MC_ROCM_BLOCKS_PER_CU,
 * XCCL_MC_ROCM_RESIDENT_PER_CU), read once at first launch.
 */
void xccl_rocm_set_launch_shape(int blocks_per_cu, int resident_per_cu);

/*
 * Launches of at most `max_grid` workgroups with four or more sources run the
 * burst kernel (every load of a tile issued at once: such a launch is bound by
 * latency, not by bandwidth); larger ones walk their sources two loads at a
 * time.  Same results either way.  0 = never, negative = the built-in default;
 * also XCCL_MC_ROCM_BURST_MAX_GRID.  For measurement and tests.
 */
void xccl_rocm_set_burst_max_grid(int max_grid);

/* Largest launch, in workgroups, that reports completion on one word per
 * workgroup (xccl_rocm_reduce_multi_slots); 0 = never, negative = the built-in
 * default (8).  For measurement and tests. */
void xccl_rocm_set_slot_max_grid(int max_grid);

/* Largest launch, in workgroups, that counts its own arrivals for the
 * completion word: on a HIP stream (default 2048; larger ones get a one-lane
 * kernel queued behind them) and on the component's own queue (default 64;
 * 6144 with the second packet of xccl_rocm_set_direct_tail switched off).
 * Negative = leave alone.  Also XCCL_MC_ROCM_MAX_COUNTED_GRID (sets both).
 * For measurement and tests. */
void xccl_rocm_set_counted_grid(int on_stream, int on_own_queue);

/* What a launch with these arguments would be: grid/block size and the
 * mangled kernel name (truncated into `name`, if not NULL).  Host-only apart
 * from the CU-count query.  Returns the status the launch would return. */
xccl_status_t xccl_rocm_reduce_multi_plan(void *sbuf1, void *sbuf2, void *rbuf,
                                          size_t count, size_t size,
                                          size_t stride, xccl_dt_t dtype,
                                          xccl_op_t op, unsigned *grid,
                                          unsigned *block, char *name,
                                          size_t name_len);

/* What a launch with these arguments, asked to report its own completion,
 * would be -- on a HIP stream (`own_queue` 0) or on the component's own queue
 * (1): grid in workgroups, bytes of LDS asked for to bound the resident
 * workgroups per compute unit (0: no bound), whether it runs the burst
 * kernel, and how the host learns that it is complete.  Any output may be
 * NULL.  Host-only apart from the CU-count query; every launch-shape knob and
 * its environment variable shows here.  For tests. */
enum {
    XCCL_ROCM_ROUTE_STREAM  = 0, /* no completion word: the caller waits for the stream */
    XCCL_ROCM_ROUTE_SLOTS   = 1, /* one word per workgroup */
    XCCL_ROCM_ROUTE_COUNTED = 2, /* the last workgroup to arrive writes the word */
    XCCL_ROCM_ROUTE_TAIL    = 3, /* a one-lane kernel queued behind the launch writes it */
    XCCL_ROCM_ROUTE_SIGNAL  = 4  /* the packet's completion signal (own queue only) */
};
xccl_status_t xccl_rocm_reduce_multi_route(void *sbuf1, void *sbuf2, void *rbuf,
                                           size_t count, size_t size,
                                           size_t stride, xccl_dt_t dtype,
                                           xccl_op_t op, int own_queue,
                                           unsigned *grid, unsigned *lds_bytes,
                                           int *burst, int *route);

/*
 * Stream gate used by start/finish_stream_activity: one wave polls the
 * host-mapped word at `dev_flag` until it is non-zero, or until `max_ns`
 * nanoseconds have passed (then it stores 2 to `dev_flag` itself and exits:
 * a gate the host never opens cannot hang the queue).
 * Replaces xccl_cuda_dummy_kernel (xccl_cuda_kernel.cu:4-20), which spins
 * without a bound.
 */
xccl_status_t xccl_rocm_stream_gate(int *dev_flag, uint64_t max_ns,
                                    void *hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* XCCL_ROCM_KERNELS_H_ */
