/*
 * xccl_rocm_ucx_replay.h -- libxccl_ucx_replay.so: the reduction call sites
 * of XCCL's UCX team library, replayed in ONE process over ONE GPU.
 *
 * The UCX team library's allreduce / reduce algorithms are host state
 * machines that exchange vectors over UCP tag send/recv and, between rounds,
 * call xccl_mem_component_reduce / _reduce_multi on what arrived (reference
 * src/team_lib/ucx/allreduce/allreduce_knomial.c, allreduce_sra.c,
 * src/team_lib/ucx/reduce/reduce_knomial.c, reduce_linear.c).  UCX is not
 * part of this build, so this library keeps the algorithms' structure --
 * peers, message sizes, scratch layout, buffer aliasing, call order -- and
 * swaps the wire for a loopback: every "rank" is a set of buffers on the same
 * GPU, a matched send/recv pair is one xccl_mem_component_memcpy_async on a
 * transport stream, completion is an xccl_mc_event.  All P ranks are
 * progressed round-robin by the caller's thread, each through a resumable
 * progress function, as xccl_collective_test does for real requests.
 *
 * What is new relative to the reference: with XCCL_REPLAY_REDUCE_STREAM_ORDERED
 * a reduction is LAUNCHED (reduce_nb / reduce_multi_nb on the component
 * stream), the state machine saves a "reduce in flight" phase and returns;
 * on re-entry it polls the event and only then posts the sends that read the
 * result.  With XCCL_REPLAY_REDUCE_BLOCKING it calls the synchronous entries
 * exactly like the reference does.
 *
 * Buffers are device pointers of memory type UCS_MEMORY_TYPE_ROCM; the
 * dispatcher (libxccl_mc.so) must have been initialised with the ROCm
 * component loaded.
 */
#ifndef XCCL_ROCM_UCX_REPLAY_H_
#define XCCL_ROCM_UCX_REPLAY_H_

#include "xccl_rocm_types.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    XCCL_REPLAY_ALLREDUCE_KNOMIAL = 0, /* allreduce_knomial.c (alg 0: len < 4096 by default) */
    XCCL_REPLAY_ALLREDUCE_SRA     = 1, /* allreduce_sra.c: scatter-reduce + allgather */
    XCCL_REPLAY_REDUCE_KNOMIAL    = 2, /* reduce_knomial.c */
    XCCL_REPLAY_REDUCE_LINEAR     = 3  /* reduce_linear.c */
} xccl_replay_alg_t;

typedef enum {
    XCCL_REPLAY_REDUCE_BLOCKING       = 0,
    XCCL_REPLAY_REDUCE_STREAM_ORDERED = 1
} xccl_replay_reduce_mode_t;

typedef struct xccl_replay_params {
    xccl_replay_alg_t         alg;
    xccl_replay_reduce_mode_t reduce_mode;
    int                       team_size; /* P >= 1 */
    int                       radix;     /* k-nomial radix (reference default 4); clipped to P */
    int                       root;      /* rooted algorithms only */
    size_t                    count;     /* elements per rank */
    xccl_dt_t                 dtype;
    xccl_op_t                 op;
    void                    **src;       /* [P] device pointers, count elements each */
    void                    **dst;       /* [P] device pointers (reduce: only dst[root] is written);
                                            dst[r] == src[r] requests the in-place form */
} xccl_replay_params_t;

typedef struct xccl_replay_stats {
    uint64_t reduce_calls;        /* 2-source reductions issued */
    uint64_t reduce_multi_calls;  /* multi-source reductions issued */
    uint64_t max_multi_vectors;   /* largest `count` passed to reduce_multi */
    uint64_t inplace_sbuf1;       /* reductions with rbuf == sbuf1 */
    uint64_t inplace_sbuf2;       /* reductions with rbuf/target == sbuf2 */
    uint64_t messages;            /* matched send/recv pairs */
    uint64_t bytes_moved;         /* bytes copied by the loopback transport */
    uint64_t progress_calls;      /* total progress-function entries over all ranks */
    uint64_t reduce_inflight_returns; /* times a rank returned with its reduction still running */
    uint64_t scratch_allocs;      /* xccl_mem_component_alloc calls */
} xccl_replay_stats_t;

/* Runs one collective to completion on all ranks.  Returns XCCL_OK, the first
 * error status of a mem-component call, XCCL_ERR_INVALID_PARAM for bad
 * parameters, or XCCL_ERR_NO_PROGRESS if the ranks stop making progress
 * (`max_sweeps` round-robin sweeps without completion; 0 = default limit). */
xccl_status_t xccl_replay_run(const xccl_replay_params_t *params, xccl_replay_stats_t *stats, uint64_t max_sweeps);

/* Geometry of the recursive k-nomial exchange (allreduce_knomial.h:10-34):
 * number of exchange rounds, ranks taking part in them (`full_size`), and the
 * role of `rank`: 0 = base, 1 = proxy (also folds one extra rank's vector in
 * before round 0), 2 = extra (hands its vector to rank - full_size and waits
 * for the result).  Host-only. */
void xccl_replay_knomial_geometry(int radix, int rank, int team_size, int *rounds, int *full_size, int *role);

/* Final segment (element offset and length) that `rank` owns after the
 * scatter-reduce phase (allreduce_sra.c:77-127).  Host-only. */
void xccl_replay_sra_segment(size_t count, int rank, int radix, int team_size, size_t *offset, size_t *length);

#ifdef __cplusplus
}
#endif
#endif /* XCCL_ROCM_UCX_REPLAY_H_ */
